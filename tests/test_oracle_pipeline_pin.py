"""Numeric pins of ``oracle.pipeline_oracle.run_pipeline`` that do not go through the oracle's
own output.  CPU only.

(i)  With every warm-up depth 0 a pipeline is ordinary minibatch SGD on the unsplit model
     (one weight version, forward and backward of minibatch k back to back): the oracle must
     equal, bit for bit, an ``nn.Sequential`` of the same layers trained by plain
     ``torch.optim.SGD`` / ``Adam``.
(ii) With warm-up depths S-1-s the oracle must equal, bit for bit, a loop written from the
     definition of weight stashing instead of from the reference's mechanism: every stage
     keeps a ``deepcopy`` of its module per weight version, minibatch k runs forward AND
     backward through copy ``max(0, k - W_s)``, and the gradient is applied to the newest
     weights (runtime/image_classification/main_with_runtime.py:359-421; hand-off contract
     runtime/communication.py:595-596, 699).  No deque, no load/store of state dicts, no
     in-flight FIFO on that side.
(iii) Mutants of ``run_pipeline`` (a dropped ``.detach()``, the newest instead of the oldest
     version loaded for backward, LIFO instead of FIFO, a gradient sent to the wrong
     neighbour, a missing ``requires_grad_``) must each fail (i) or (ii): the pins see the
     mistakes they are there for."""
import copy
import inspect
import textwrap

import pytest
import torch

from oracle import pipeline_oracle, stash_oracle as so

SGD_KW = dict(lr=0.05, momentum=0.9, weight_decay=1e-3)
ADAM_KW = dict(lr=0.01, betas=(0.9, 0.99), weight_decay=1e-3)


def _stages(S, seed=0):
    torch.manual_seed(seed)
    if S == 2:
        blocks = [[torch.nn.Linear(6, 8), torch.nn.ReLU(), torch.nn.Linear(8, 8), torch.nn.Tanh()],
                  [torch.nn.Linear(8, 4)]]
    else:
        blocks = [[torch.nn.Linear(6, 8), torch.nn.ReLU()],
                  [torch.nn.Linear(8, 8), torch.nn.Tanh(), torch.nn.Linear(8, 7), torch.nn.ReLU()],
                  [torch.nn.Linear(7, 4)]]
    return [torch.nn.Sequential(*b) for b in blocks]


def _batches(n, seed=1):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(5, 6, generator=g), torch.randint(0, 4, (5,), generator=g)) for _ in range(n)]


def _make_opt(name, kw):
    return lambda s, m, nv: so.StashingOptimizerOracle(name, [m], m.parameters(), nv, **kw)


def _run_oracle(run_pipeline, S, n, name, kw, warmups):
    stages = _stages(S)
    losses, st = run_pipeline(stages, torch.nn.CrossEntropyLoss(), _make_opt(name, kw), _batches(n), warmups=warmups)
    return losses, [copy.deepcopy(m.state_dict()) for m in stages], st


def _unsplit(S, n, name, kw):
    """The same layers as one model under the library's own optimizer."""
    stages = _stages(S)
    model = torch.nn.Sequential(*stages)
    opt = getattr(torch.optim, name)(model.parameters(), **kw)
    crit = torch.nn.CrossEntropyLoss()
    losses = []
    for x, y in _batches(n):
        opt.zero_grad()
        loss = crit(model(x), y)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
    return losses, [copy.deepcopy(m.state_dict()) for m in stages]


def _versioned_copies(S, n, name, kw):
    """Weight stashing from its definition.  Iteration k: minibatch k goes forward through every
    stage on that stage's copy of version max(0, k - W_s); then stage s (last first) runs the
    backward pass of minibatch k - W_s through the very copy that its forward used and applies the
    gradient to the stage's newest weights, which creates the next version."""
    newest = _stages(S)
    W = [S - 1 - s for s in range(S)]
    opts = [getattr(torch.optim, name)(m.parameters(), **kw) for m in newest]
    versions = [{0: copy.deepcopy(m)} for m in newest]
    crit = torch.nn.CrossEntropyLoss()
    batches = _batches(n)
    graph = {}        # (stage, minibatch) -> (stage input, stage output or loss, module copy used)
    grads = {}        # (stage, minibatch) -> gradient w.r.t. that stage's output
    losses = [None] * n

    def backward(s, j):
        x, out, used = graph.pop((s, j))
        for p in used.parameters():
            p.grad = None
        if s == S - 1:
            out.backward()
        else:
            out.backward(grads.pop((s, j)))
        if s > 0:
            grads[(s - 1, j)] = x.grad
        for p_new, p_used in zip(newest[s].parameters(), used.parameters()):
            p_new.grad = p_used.grad
        opts[s].step()
        versions[s][j + 1] = copy.deepcopy(newest[s])
        for p in versions[s][j + 1].parameters():
            p.grad = None
        versions[s].pop(j - W[s] - 1, None)

    for k in range(n + S - 1):
        if k < n:
            x, y = batches[k]
            for s in range(S):
                used = versions[s][max(0, k - W[s])]
                if s > 0:
                    x = x.detach().requires_grad_()
                out = used(x)
                if s == S - 1:
                    out = crit(out, y)
                    losses[k] = float(out.detach())
                graph[(s, k)] = (x, out, used)
                x = out
        for s in reversed(range(S)):
            j = k - W[s]
            if 0 <= j < n:
                backward(s, j)
    assert not graph and not grads
    return losses, [copy.deepcopy(m.state_dict()) for m in newest]


def _assert_same(a, b):
    la, pa = a[0], a[1]
    lb, pb = b[0], b[1]
    assert la == lb, (la, lb)
    for sa, sb in zip(pa, pb):
        assert sa.keys() == sb.keys()
        for k in sa:
            assert torch.equal(sa[k], sb[k]), k


@pytest.mark.parametrize("S", [2, 3])
@pytest.mark.parametrize("name,kw", [("SGD", SGD_KW), ("Adam", ADAM_KW)])
def test_zero_warmup_equals_unsplit_model(S, name, kw):
    got = _run_oracle(pipeline_oracle.run_pipeline, S, 12, name, kw, [0] * S)
    _assert_same(got, _unsplit(S, 12, name, kw))
    for st in got[2]:
        assert st.fwd_versions == st.bwd_versions == list(range(12))


@pytest.mark.parametrize("S", [2, 3])
@pytest.mark.parametrize("name,kw", [("SGD", SGD_KW), ("Adam", ADAM_KW)])
def test_stashed_pipeline_equals_versioned_copies(S, name, kw):
    n = 11
    got = _run_oracle(pipeline_oracle.run_pipeline, S, n, name, kw, None)
    _assert_same(got, _versioned_copies(S, n, name, kw))
    for s, st in enumerate(got[2]):
        want = [max(0, k - (S - 1 - s)) for k in range(n)]
        assert st.fwd_versions == want and st.bwd_versions == want


def test_stashing_is_not_a_no_op_here():
    """The two pins would be worthless on a problem where the version does not matter: the
    stashed run must differ from the unsplit one."""
    a = _run_oracle(pipeline_oracle.run_pipeline, 3, 11, "SGD", SGD_KW, None)
    b = _unsplit(3, 11, "SGD", SGD_KW)
    assert a[0][:1] == b[0][:1] and a[0][3:] != b[0][3:]


def test_lr_schedule_hook_equals_unsplit_model_with_per_step_lr():
    """The oracle's learning-rate hook against the unsplit model whose ``param_group['lr']`` is written
    before every step (main_with_runtime.py:368, 562-563)."""
    lrs = [0.01 * (1 + i) for i in range(10)]
    stages = _stages(2)
    losses, _ = pipeline_oracle.run_pipeline(stages, torch.nn.CrossEntropyLoss(), _make_opt("SGD", SGD_KW),
                                             _batches(10), warmups=[0, 0], lr_schedule=lambda s, i: lrs[i])
    ref = _stages(2)
    model = torch.nn.Sequential(*ref)
    opt = torch.optim.SGD(model.parameters(), **SGD_KW)
    crit = torch.nn.CrossEntropyLoss()
    ref_losses = []
    for i, (x, y) in enumerate(_batches(10)):
        loss = crit(model(x), y)
        for g in opt.param_groups:
            g["lr"] = lrs[i]
        opt.zero_grad()
        loss.backward()
        opt.step()
        ref_losses.append(float(loss.detach()))
    _assert_same((losses, [m.state_dict() for m in stages]), (ref_losses, [m.state_dict() for m in ref]))
    # with a warm-up depth the first W forwards leave the rate alone: stage 0 applies lrs[i] to its i-th update
    seen = []
    stages = _stages(2)
    pipeline_oracle.run_pipeline(stages, torch.nn.CrossEntropyLoss(), _make_opt("SGD", SGD_KW), _batches(6),
                                 lr_schedule=lambda s, i: seen.append((s, i)) or lrs[i])
    assert [i for s, i in seen if s == 0] == list(range(5)) and [i for s, i in seen if s == 1] == list(range(6))


def _mutant(old, new):
    src = textwrap.dedent(inspect.getsource(pipeline_oracle.run_pipeline))
    assert src.count(old) == 1, old
    scope = dict(vars(pipeline_oracle))
    exec(compile(src.replace(old, new), "<mutant>", "exec"), scope)
    return scope["run_pipeline"]


MUTANTS = [
    ("fwd_q[s + 1].append(out.detach())", "fwd_q[s + 1].append(out)"),
    ("opt.load_old_params()", "opt.load_new_params()"),
    ("x, out = st.in_flight.popleft()", "x, out = st.in_flight.pop()"),
    ("x = x.requires_grad_()", "x = x"),
    ("bwd_q[s - 1].append(x.grad)", "bwd_q[s - 1].append(x.grad * 1.0000002)"),
    ("opt.load_new_params()\n", "pass\n"),
]


@pytest.mark.parametrize("old,new", MUTANTS)
def test_mutants_fail_a_pin(old, new):
    mutant = _mutant(old, new)
    failed = False
    for check in (lambda: _assert_same(_run_oracle(mutant, 3, 9, "SGD", SGD_KW, [0, 0, 0]), _unsplit(3, 9, "SGD", SGD_KW)),
                  lambda: _assert_same(_run_oracle(mutant, 3, 9, "SGD", SGD_KW, None),
                                       _versioned_copies(3, 9, "SGD", SGD_KW))):
        try:
            check()
        except (AssertionError, RuntimeError, TypeError, IndexError):
            failed = True
    assert failed, "mutant survived both pins: %s" % new
