"""CPU ORACLE -- test infrastructure, not product code.

A multi-stage 1F1B pipeline with weight stashing on CPU ``torch.nn`` modules: the
behaviour of N reference processes (runtime/image_classification/main_with_runtime.py:
333-427 driving runtime/runtime.py:488-624 and runtime/optimizer.py) replayed in one
process.  Used by tests/ and bench.py's cpu_baseline leg as the checker / the timed
CPU path; never imported by ``pipedream_amd``.

Stage compute is the installed torch library on CPU (``torch.nn`` modules +
``torch.autograd.backward``), which is what the reference's generated stage modules call
(third-party arithmetic; the reference pins PyTorch 1.1, README.md:50).  The hand-off
contract is the reference's: a forward-received fp32 tensor becomes a leaf that
requires grad (runtime/communication.py:595-596), what is sent is detached (:699), and
backward pops the oldest in-flight minibatch (runtime/runtime.py:571).

How ``run_pipeline`` is pinned (tests/test_oracle_pipeline_pin.py, tests/test_pipeline_mlp.py): its
event order against the closed form of the 1F1B loop; its numbers, bit for bit, (i) with all
warm-up depths 0 against the unsplit ``nn.Sequential`` under the library's ``torch.optim.SGD`` /
``Adam``, and (ii) with depths S-1-s against a loop written from the definition of weight stashing
(one ``deepcopy`` of a stage per version, forward and backward of minibatch k through copy
``max(0, k - W)``); mutants of this function (dropped ``detach``, wrong version, LIFO, missing
leaf, perturbed hand-off gradient) fail those pins.
"""
import collections

import torch

from . import stash_oracle as so


# dtypes that become gradient-requiring leaves on receipt (runtime/communication.py:595)
LEAF_DTYPES = (torch.float32,)


class StageOracle(object):
    def __init__(self, module, optimizer, warmup, is_last, criterion=None, loss_scale=1.0):
        self.module = module
        self.optimizer = optimizer
        self.warmup = warmup
        self.is_last = is_last
        self.criterion = criterion
        self.loss_scale = loss_scale
        self.in_flight = collections.deque()
        self.fwd_versions = []
        self.bwd_versions = []


def run_pipeline(stage_modules, criterion, make_optimizer, batches, warmups=None, on_loss=None, lr_schedule=None,
                 observer=None):
    """Run ``len(batches)`` minibatches through the stages with 1F1B + weight stashing.

    ``stage_modules``: CPU modules, stage 0 first; ``make_optimizer(stage_index, module,
    num_versions)`` returns a ``StashingOptimizerOracle``; ``batches``: list of
    ``(input, target)``; ``warmups``: warm-up depth per stage (default: straight pipeline,
    S-1-s); ``lr_schedule(stage_index, i)``: learning rate written into every param group after
    the i-th steady-state forward of a stage, as ``adjust_learning_rate`` is called at
    main_with_runtime.py:368 (warm-up forwards do not touch it); ``observer(kind, s, k, **tensors)``
    is shown every pass without taking part in it: ``("F", x, target, out)`` after a forward pass (``out``
    is the loss on the last stage) and ``("B", grad_out, grad_in, stage)`` after a backward pass and its
    update (``grad_out`` None on the last stage, ``grad_in`` None on the first).
    Returns (losses in minibatch order, list of StageOracle)."""
    S = len(stage_modules)
    n = len(batches)
    if warmups is None:
        warmups = [so.warmup_depth(s, {i: [i] for i in range(S)}) for s in range(S)]
    stages = []
    for s, m in enumerate(stage_modules):
        stages.append(StageOracle(m, make_optimizer(s, m, warmups[s] + 1), warmups[s], s == S - 1, criterion))
        m.train()
    events = [collections.deque(so.one_f_one_b(n, w)) for w in warmups]
    fwd_q = [collections.deque() for _ in range(S + 1)]   # fwd_q[s]: activations waiting for stage s
    bwd_q = [collections.deque() for _ in range(S + 1)]   # bwd_q[s]: output grads waiting for stage s
    tgt_q = [collections.deque() for _ in range(S + 1)]
    losses = {}

    def runnable(s):
        kind, k = events[s][0]
        if kind == "F":
            return s == 0 or len(fwd_q[s]) > 0
        return stages[s].is_last or len(bwd_q[s]) > 0

    while any(events):
        progressed = False
        for s in range(S):
            while events[s] and runnable(s):
                kind, k = events[s].popleft()
                st = stages[s]
                progressed = True
                if kind == "F":
                    if s == 0:
                        x, target = batches[k]
                    else:
                        x = fwd_q[s].popleft()
                        target = tgt_q[s].popleft()
                        if x.dtype in LEAF_DTYPES:
                            x = x.requires_grad_()
                    st.fwd_versions.append(st.optimizer.latest_version)
                    out = st.module(x)
                    if st.is_last:
                        loss = criterion(out, target)
                        losses[k] = float(loss.detach())
                        if on_loss is not None:
                            on_loss(k, losses[k])
                        st.in_flight.append((x, loss))
                    else:
                        st.in_flight.append((x, out))
                        fwd_q[s + 1].append(out.detach())
                        tgt_q[s + 1].append(target)
                    if observer is not None:
                        observer("F", s, k, x=x, target=target, out=st.in_flight[-1][1])
                    if lr_schedule is not None and k >= min(st.warmup, n):
                        for group in st.optimizer.param_groups:
                            group["lr"] = lr_schedule(s, k - min(st.warmup, n))
                else:
                    opt = st.optimizer
                    opt.zero_grad()
                    opt.load_old_params()
                    st.bwd_versions.append(opt.current_version if opt.num_versions > 1 else opt.latest_version)
                    x, out = st.in_flight.popleft()
                    grad_out = None
                    if st.is_last:
                        (out * st.loss_scale).backward()
                    else:
                        grad_out = bwd_q[s].popleft()
                        torch.autograd.backward((out,), grad_tensors=(grad_out,))
                    if s > 0:
                        bwd_q[s - 1].append(x.grad)
                    opt.load_new_params()
                    opt.step()
                    if observer is not None:
                        observer("B", s, k, grad_out=grad_out, grad_in=x.grad if s > 0 else None, stage=st)
        if not progressed:
            raise RuntimeError("oracle pipeline deadlocked")
    return [losses[k] for k in range(n)], stages
