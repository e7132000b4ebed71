"""``OptimizerWithWeightStashing`` with the reference's API over the HBM version ring.

Mirror of runtime/optimizer.py in the reference (class ``Version`` :9-17, class
``OptimizerWithWeightStashing`` :19-164): same constructor, same methods
(``zero_grad``, ``load_old_params``, ``load_new_params``, ``step``, ``get_params``,
``set_params``, ``initialize_queue``), same attributes (``queue``, ``latest_version``,
``current_version``, ``num_versions``, ``update_interval``, ``batch_counter``), and every
other attribute is relayed to the base optimizer.

What differs is where the bytes live.  The reference keeps ``num_versions`` cloned
``state_dict``s plus the live module and moves 3 full copies per step with per-tensor
``copy_`` calls.  Here the versions are slots of one flat device buffer, the live
module tensors are views of the loaded slot (so loading is a pointer swap), and the
optimizer step reads the newest slot and writes the oldest slot's storage in the same
fused kernel that applies the update.
"""
import collections
import time

import torch

from . import _cabi
from .arena import WeightArena
from .fused_optim import BASE_OPTIMIZERS


class Version(object):
    """runtime/optimizer.py:9-17"""

    def __init__(self, version=0):
        self.version = version

    def __repr__(self):
        return "v%d" % self.version

    def __eq__(self, other):
        return isinstance(other, Version) and other.version == self.version

    def __hash__(self):
        return hash(self.version)

    def incr(self):
        return Version(version=self.version + 1)


def prep_param_lists(model):
    """``(model parameters, fp32 master parameters)`` of a 16-bit module: what runtime/runtime.py:268-276
    obtains from ``apex.fp16_utils.prep_param_lists`` (third-party, not needed here): the module's own
    parameters and, for each, a detached fp32 clone that requires grad."""
    model_params = [p for p in model.parameters() if p.requires_grad]
    master_params = [p.detach().clone().float().requires_grad_() for p in model_params]
    return model_params, master_params


class _RingQueue(object):
    """Read-only ``deque``-like face of the ring: ``queue[i] -> (state_dicts, Version)``
    with index 0 the oldest entry, as ``deque(maxlen=num_versions)`` in the reference."""

    def __init__(self, arena):
        self._arena = arena

    def __len__(self):
        return self._arena.num_versions

    def __getitem__(self, i):
        slot, version = self._arena.entry(i)
        return self._arena.state_dicts(slot), Version(version)

    def __iter__(self):
        for i in range(len(self)):
            yield self[i]

    @property
    def maxlen(self):
        return self._arena.num_versions

    def versions(self):
        """[version held by queue[0], ..., queue[-1]] (integers)."""
        return [self._arena.entry(i)[1] for i in range(len(self))]

    def slots(self):
        return [self._arena.entry(i)[0] for i in range(len(self))]


class OptimizerWithWeightStashing(torch.optim.Optimizer):
    """Wrapper that adds weight stashing to a fused base optimizer.

    Arguments are those of the reference (runtime/optimizer.py:28-30).  ``optim_name``
    selects the base optimizer: ``'SGD'`` or ``'Adam'`` (the two the reference's
    runtime/sgd.py and runtime/adam.py use).  ``update_interval`` (not in the
    reference) decouples gradient accumulation from ``num_versions`` for 2BW-style
    double buffering; left at ``None`` it follows the reference rule.  ``bf16_image`` (not
    in the reference) keeps a bf16 copy of every weight version for bf16-compute stages.

    ``model_parameters`` (the reference's fp16 arrangement, optimizer.py:137-155): the modules hold 16-bit
    parameters (bfloat16 or float16), ``master_parameters`` are their fp32 masters (``prep_param_lists``).
    The ring then stashes the 16-bit versions, and a step -- model gradients widened to fp32, divided by
    ``loss_scale``, the base optimizer on the masters, the masters copied back into the model -- is the same
    single launch, which reads the 16-bit gradients and writes the 16-bit image of the new weights into
    the ring's write slot.
    """

    def __init__(self, optim_name, modules, master_parameters, model_parameters,
                 loss_scale, num_versions, verbose_freq=0, macrobatch=False,
                 update_interval=None, bf16_image=False, **optimizer_args):
        if optim_name not in BASE_OPTIMIZERS:
            raise NotImplementedError(
                "optim_name %r has no fused HIP kernel (available: %s)" % (optim_name, sorted(BASE_OPTIMIZERS)))
        if model_parameters is not None:
            # mixed precision (optimizer.py:137-155): 16-bit parameters in the modules, fp32 masters beside them
            model_parameters = list(model_parameters)
        self.modules = modules
        self.master_parameters = master_parameters = list(master_parameters)
        self.model_parameters = model_parameters
        self.loss_scale = loss_scale

        # Only need at most 2 versions if using macrobatching (optimizer.py:36-38).
        if macrobatch:
            num_versions = min(2, num_versions)
        self.num_versions = num_versions

        flat_masters = []
        for item in master_parameters:
            if isinstance(item, dict):
                flat_masters.extend(item["params"])
            else:
                flat_masters.append(item)
        self.arena = WeightArena(self.modules, flat_masters, num_versions, bf16_image=bf16_image,
                                 model_parameters=model_parameters)
        self.base_optimizer = BASE_OPTIMIZERS[optim_name](master_parameters, arena=self.arena, **optimizer_args)
        self.latest_version = Version()
        self.current_version = Version()
        self.initialize_queue()
        self.verbose_freq = verbose_freq
        self.batch_counter = 0

        # If macrobatching, push and pop versions at the right rate (optimizer.py:48-52).
        if update_interval is not None:
            self.update_interval = int(update_interval)
        elif macrobatch:
            self.update_interval = self.num_versions
        else:
            self.update_interval = 1

    def __getattr__(self, key):
        """Relay the unknown key to base_optimizer (optimizer.py:54-56)."""
        if key in ("base_optimizer", "arena"):
            raise AttributeError(key)
        return getattr(self.base_optimizer, key)

    # state / param_groups of torch.optim.Optimizer are never initialised on the wrapper
    # (the reference does not call super().__init__ either); they resolve via __getattr__.

    def initialize_queue(self):
        """The arena already holds ``num_versions`` clones at version 0
        (optimizer.py:58-62); expose them with the reference's deque interface."""
        self.queue = _RingQueue(self.arena)

    @property
    def buffered_state_dicts(self):
        """Views of the storage the next step overwrites (optimizer.py:62, :157)."""
        return self.queue[0][0]

    def state_dict(self):
        return self.base_optimizer.state_dict()

    def load_state_dict(self, state_dict):
        return self.base_optimizer.load_state_dict(state_dict)

    def get_params(self, clone):
        """optimizer.py:64-85."""
        if clone:
            state_dicts = []
            for module in self.modules:
                state_dict = module.state_dict()
                for key in state_dict:
                    state_dict[key] = state_dict[key].clone()
                state_dicts.append(state_dict)
        else:
            # live values -> storage of the oldest entry
            dst = self.arena.write_slot()
            self.arena.copy_masters(self.arena.live_slot, dst)
            self.arena.refresh_bf16_image(dst)
            self.arena.store_others(dst)
            state_dicts = self.arena.state_dicts(dst)
        return state_dicts, self.latest_version

    def set_params(self, state_dicts, version):
        """optimizer.py:87-108.  A stash produced by this class is loaded by pointing the
        module tensors at its slot; foreign state_dicts are copied into the loaded slot."""
        slot = getattr(state_dicts[0], "_pd_slot", None) if len(state_dicts) else None
        if slot is not None and all(getattr(d, "_pd_slot", None) == slot for d in state_dicts):
            self.arena.load_slot(slot)
        else:
            with torch.no_grad():
                for (state_dict, module) in zip(state_dicts, self.modules):
                    cur = module.state_dict()
                    for key in state_dict:
                        if "running_" in key or "mask" in key:
                            continue
                        cur[key].copy_(state_dict[key])
            # the copy went into the loaded slot's fp32 masters; bf16-compute layers read its bf16 image
            self.arena.refresh_bf16_image()
        self.current_version = version

    def load_old_params(self):
        if self.num_versions > 1:
            slot, version = self.arena.entry(0)
            self.arena.load_slot(slot)
            self.current_version = Version(version)

    def load_new_params(self):
        if self.num_versions > 1:
            slot, version = self.arena.entry(-1)
            self.arena.load_slot(slot)
            self.current_version = Version(version)

    def zero_grad(self, set_to_none=True):
        if self.batch_counter % self.update_interval == 0:
            self.base_optimizer.zero_grad(set_to_none=set_to_none)

    def step(self, closure=None):
        """Performs a single optimization step (optimizer.py:122-164).

        The gradient scaling (``/ loss_scale``, ``/ update_interval``), the base
        optimizer's update and the copy of the new weights into the oldest ring entry
        are one kernel launch; unlike the reference the gradients themselves are left
        unscaled in ``p.grad`` afterwards.
        """
        # Update the gradient every `update_interval` steps.
        if self.batch_counter % self.update_interval != self.update_interval - 1:
            self.batch_counter += 1
            return None

        log_timing = self.verbose_freq > 0 and self.batch_counter % self.verbose_freq == 0
        if log_timing:
            start_time = time.time()

        arena = self.arena
        in_slot = arena.live_slot
        out_slot = arena.write_slot() if self.num_versions > 1 else in_slot
        # the reference divides by loss_scale only on the mixed-precision branch (optimizer.py:137-145)
        loss_scale = float(self.loss_scale) if self.model_parameters is not None else 1.0
        loss = self.base_optimizer.step(closure, in_slot=in_slot, out_slot=out_slot,
                                        loss_scale=loss_scale, update_interval=float(self.update_interval))
        self.latest_version = self.latest_version.incr()
        if self.num_versions > 1:
            arena.store_others(out_slot)
            pushed = arena.push(self.latest_version.version)
            assert pushed == out_slot
            arena.load_slot(out_slot, with_others=False)

        if log_timing:
            print("Optimizer step took: %.3f" % (time.time() - start_time))
        self.batch_counter += 1
        return loss
