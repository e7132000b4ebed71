"""CPU ORACLE -- test infrastructure, not product code.

A CPU restatement of the reference's per-stage training step, used only by ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` as the checker
(never imported by ``pipedream_amd``).

What is restated, and from where (paths relative to the reference checkout):

* ``StashingOptimizerOracle``  -- runtime/optimizer.py:19-164: a ``deque(maxlen=nv)`` of
  cloned per-module ``state_dict``s paired with a version number; ``load_old_params`` /
  ``load_new_params`` copy ``queue[0]`` / ``queue[-1]`` into the live module, skipping
  ``running_*`` and ``mask`` keys; ``step`` divides the gradients by ``update_interval``,
  runs the base optimizer, then copies the live state into the oldest entry's storage
  and re-appends it.  The copies go through ``.data.copy_`` because
  ``Module.load_state_dict`` (an in-place write under autograd's eyes) is rejected by
  torch >= 1.5 while a minibatch is in flight; PyTorch 1.1, which the reference pins
  (README.md:50), wrote through ``.data`` as well.
* ``sgd_step_numpy`` / ``adam_step_numpy`` -- the arithmetic of the third-party
  optimizers the reference selects by name (runtime/sgd.py:17, runtime/adam.py:16,
  constructed at runtime/optimizer.py:40-41): ``torch.optim.SGD`` and ``torch.optim.Adam``.
  These live in PyTorch, not in the reference tree; the reference pins
  ``nvcr.io/nvidia/pytorch:19.05-py3`` (PyTorch 1.1.0a0).  The restatement follows the
  published algorithm of the installed torch 2.10 (``_single_tensor_sgd`` /
  ``_single_tensor_adam``); ``eps_mode=1`` gives PyTorch 1.1's Adam
  (``denom = sqrt(v) + eps``, ``step_size = lr*sqrt(bc2)/bc1``).
* ``forward_version`` / ``backward_version`` / ``ring_versions_after`` -- the version
  selection rule that emerges from the 1F1B loop of
  runtime/image_classification/main_with_runtime.py:359-421 driving the ring.
* ``one_f_one_b`` -- the per-stage event order of that loop.
* ``warmup_depth`` -- runtime/runtime.py:162-175.
* ``adjust_learning_rate`` -- runtime/image_classification/main_with_runtime.py:532-563.

  Its mixed-precision branch (:137-155, ``model_parameters``) includes the two routines of
  apex.fp16_utils it calls, restated from their published behaviour (apex is a third-party dependency that
  is not in the reference tree: model gradients copied into fp32 master gradients, masters copied back
  into the 16-bit model); pinned by hand values in tests/test_oracle_optim.py.

How each piece is pinned (tests/test_oracle_*.py): the truth table of
runtime/tests/backprop/sgd_with_stashing.py:68-70 is reproduced on
``StashingOptimizerOracle``; the numpy optimizers are checked against the installed
``torch.optim`` library on random vectors and against hand-computed closed forms; the
version rule is checked against a brute-force ``deque`` simulation.  The reference
holds no numeric golden vectors for this path, so numeric parity is anchored on the
installed torch library ("parity unpinned by the reference" for absolute values).
"""
import collections
import math

import numpy as np
import torch


# ----------------------------------------------------------------------------------
# Version selection (integers)
# ----------------------------------------------------------------------------------
def warmup_depth(stage, stage_to_rank_map, stage_to_depth_map=None):
    """Number of warm-up forward passes of ``stage`` (runtime/runtime.py:166-175)."""
    if stage_to_depth_map is not None:
        return stage_to_depth_map[str(stage)]
    num_ranks = sum(len(r) for r in stage_to_rank_map.values())
    depth = num_ranks - 1
    for s in range(stage):
        depth -= len(stage_to_rank_map[s])
    return depth // len(stage_to_rank_map[stage])


def forward_version(k, warmup):
    """Weight version the forward pass of minibatch ``k`` (0-based) runs on."""
    return max(0, k - warmup)


def backward_version(k, warmup):
    """Weight version ``load_old_params`` loads for the backward pass of minibatch ``k``
    when ``num_versions == warmup + 1``: the same one its forward pass used."""
    return max(0, k - warmup)


def ring_versions_after(steps, num_versions):
    """Versions held by ``queue[0..nv-1]`` after ``steps`` optimizer steps."""
    return [max(0, steps - (num_versions - 1) + i) for i in range(num_versions)]


def one_f_one_b(num_minibatches, warmup):
    """Event order of one stage: list of ("F"|"B", minibatch id).
    W forwards, then (n-W) x [F, B], then W x [B]; backward order is FIFO
    (main_with_runtime.py:359-421; runtime/runtime.py:571)."""
    warmup = min(warmup, num_minibatches)
    events = [("F", i) for i in range(warmup)]
    b = 0
    for i in range(num_minibatches - warmup):
        events.append(("F", warmup + i))
        events.append(("B", b))
        b += 1
    for _ in range(warmup):
        events.append(("B", b))
        b += 1
    return events


def simulate_versions(num_minibatches, warmup, num_versions, update_interval=1):
    """Brute-force replay of the ring with integers instead of weights.
    Returns (forward versions, backward versions, final queue)."""
    queue = collections.deque(maxlen=num_versions)
    for _ in range(num_versions):
        queue.append(0)
    live = 0           # version currently loaded in the "module"
    latest = 0
    counter = 0
    fwd, bwd = {}, {}
    for kind, k in one_f_one_b(num_minibatches, warmup):
        if kind == "F":
            fwd[k] = live
        else:
            if num_versions > 1:
                live = queue[0]
            bwd[k] = live
            if num_versions > 1:
                live = queue[-1]
            if counter % update_interval == update_interval - 1:
                latest += 1
                live = latest          # base optimizer updated the live weights
                if num_versions > 1:
                    queue.append(latest)
            counter += 1
    return fwd, bwd, list(queue)


# ----------------------------------------------------------------------------------
# Optimizer arithmetic (numpy, fp32 throughout, scalars as Python doubles cast once)
# ----------------------------------------------------------------------------------
_f32 = np.float32


def sgd_step_numpy(p, g, buf, lr, momentum=0.0, dampening=0.0, weight_decay=0.0, nesterov=False):
    """One ``torch.optim.SGD`` step.  ``buf`` is None before the first step.
    Returns (new p, new buf).  Inputs are fp32 arrays and are not modified."""
    p = p.astype(_f32)
    g = g.astype(_f32)
    if weight_decay != 0:
        g = g + _f32(weight_decay) * p
    if momentum != 0:
        if buf is None:
            buf = g.copy()
        else:
            buf = buf.astype(_f32) * _f32(momentum) + _f32(1.0 - dampening) * g
        g = g + _f32(momentum) * buf if nesterov else buf
    return (p + _f32(-lr) * g).astype(_f32), buf


def adam_step_numpy(p, g, m, v, step, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, eps_mode=0):
    """One ``torch.optim.Adam`` step; ``step`` is the 1-based count of this step.
    Returns (new p, new m, new v)."""
    p = p.astype(_f32)
    g = g.astype(_f32)
    m = m.astype(_f32)
    v = v.astype(_f32)
    if weight_decay != 0:
        g = g + _f32(weight_decay) * p
    w = _f32(1.0 - beta1)
    m = m + w * (g - m)                                    # lerp_
    v = v * _f32(beta2) + (_f32(1.0 - beta2) * g) * g      # mul_ + addcmul_
    bc1 = 1.0 - beta1 ** step
    bc2 = 1.0 - beta2 ** step
    if eps_mode == 0:
        step_size = lr / bc1
        denom = np.sqrt(v) / _f32(bc2 ** 0.5) + _f32(eps)
    else:
        step_size = lr * math.sqrt(bc2) / bc1
        denom = np.sqrt(v) + _f32(eps)
    p = p + (_f32(-step_size) * m) / denom                 # addcdiv_
    return p.astype(_f32), m.astype(_f32), v.astype(_f32)


# ----------------------------------------------------------------------------------
# The weight-stashing wrapper, restated on CPU torch modules
# ----------------------------------------------------------------------------------
class StashingOptimizerOracle(object):
    """``OptimizerWithWeightStashing`` of the reference on CPU tensors."""

    def __init__(self, optim_name, modules, master_parameters, num_versions, macrobatch=False,
                 update_interval=None, model_parameters=None, loss_scale=1.0, **optimizer_args):
        """``model_parameters`` / ``loss_scale``: the mixed-precision branch (runtime/optimizer.py:137-155), with
        the two apex.fp16_utils routines it calls (third-party, absent here) restated from their published
        behaviour: ``model_grads_to_master_grads`` copies every model gradient into the fp32 gradient of its
        master, ``master_params_to_model_params`` copies every master into its (16-bit) model parameter."""
        self.model_parameters = None if model_parameters is None else list(model_parameters)
        self.loss_scale = loss_scale
        self.modules = list(modules)
        if macrobatch:
            num_versions = min(2, num_versions)
        self.num_versions = num_versions
        # The base optimizer works on ``.data`` aliases of the parameters: same storage,
        # separate autograd version counter -- what ``p.data.add_`` did in PyTorch 1.1.
        self._masters = list(master_parameters)
        self._aliases = [p.data for p in self._masters]
        self.base_optimizer = getattr(torch.optim, optim_name)(self._aliases, **optimizer_args)
        self.latest_version = 0
        self.current_version = 0
        self.queue = collections.deque(maxlen=num_versions)
        for _ in range(num_versions):
            self.queue.append((self._clone_state(), 0))
        self.batch_counter = 0
        if update_interval is not None:
            self.update_interval = update_interval      # decoupled accumulation (2BW-style)
        else:
            self.update_interval = num_versions if macrobatch else 1

    @property
    def param_groups(self):
        return self.base_optimizer.param_groups

    def _clone_state(self):
        return [collections.OrderedDict((k, t.detach().clone()) for k, t in m.state_dict().items())
                for m in self.modules]

    @staticmethod
    def _rolls_back(key):
        return "running_" not in key and "mask" not in key

    def _store_into(self, stash):
        for m, saved in zip(self.modules, stash):
            for key, t in m.state_dict().items():
                if "running_" in key:
                    continue
                if "mask" in key:
                    saved[key] = t.detach().clone()
                else:
                    saved[key].copy_(t.detach())

    def _load(self, stash, version):
        for m, saved in zip(self.modules, stash):
            live = m.state_dict()
            for key, t in saved.items():
                if self._rolls_back(key):
                    live[key].data.copy_(t)
        self.current_version = version

    def load_old_params(self):
        if self.num_versions > 1:
            self._load(*self.queue[0])

    def load_new_params(self):
        if self.num_versions > 1:
            self._load(*self.queue[-1])

    def zero_grad(self):
        if self.batch_counter % self.update_interval == 0:
            for p in self._masters:
                p.grad = None

    def step(self):
        if self.batch_counter % self.update_interval != self.update_interval - 1:
            self.batch_counter += 1
            return
        if self.model_parameters is not None:
            for model, master in zip(self.model_parameters, self._masters):      # model_grads_to_master_grads
                master.grad = None if model.grad is None else model.grad.detach().float()
            if self.loss_scale != 1.0:                                           # optimizer.py:143-145
                for master in self._masters:
                    if master.grad is not None:
                        master.grad = master.grad / self.loss_scale
        for p, alias in zip(self._masters, self._aliases):
            if p.grad is not None:
                p.grad.div_(self.update_interval)
            alias.grad = p.grad
        self.base_optimizer.step()
        if self.model_parameters is not None:
            for model, master in zip(self.model_parameters, self._masters):      # master_params_to_model_params
                model.data.copy_(master.data)
        self.latest_version += 1
        if self.num_versions > 1:
            oldest = self.queue[0][0]
            self._store_into(oldest)
            self.queue.append((oldest, self.latest_version))
        self.batch_counter += 1

    def versions(self):
        return [v for (_, v) in self.queue]


# ----------------------------------------------------------------------------------
# Learning-rate policy of the caller
# ----------------------------------------------------------------------------------
def adjust_learning_rate(stage_base_lr, epoch, total_epochs, lr_policy, step, epoch_length, lr_warmup=False):
    """main_with_runtime.py:532-563 (the value written into every param group)."""
    if lr_warmup and epoch < 5:
        return stage_base_lr * float(1 + step + epoch * epoch_length) / (5. * epoch_length)
    if lr_policy == "step":
        return stage_base_lr * (0.1 ** (epoch // 30))
    if lr_policy == "polynomial":
        return stage_base_lr * ((1.0 - (float(epoch) / float(total_epochs))) ** 2.0)
    if lr_policy == "exponential_decay":
        return stage_base_lr * (0.97 ** (float(epoch) / float(total_epochs)))
    raise NotImplementedError(lr_policy)
