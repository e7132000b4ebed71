"""LR policy (host logic, no GPU): product vs the oracle's restatement and closed forms of
runtime/image_classification/main_with_runtime.py:545-557."""
import itertools

import pytest

from oracle import stash_oracle as so
from pipedream_amd import lr_policy


def test_product_matches_oracle_everywhere():
    for policy, warm, epoch, step in itertools.product(
            ("step", "polynomial", "exponential_decay"), (False, True), (0, 3, 4, 5, 29, 30, 59, 89), (0, 7, 99)):
        a = lr_policy.learning_rate(0.04, epoch, 90, policy, step, 100, warm)
        b = so.adjust_learning_rate(0.04, epoch, 90, policy, step, 100, warm)
        assert a == b


def test_closed_forms():
    assert lr_policy.learning_rate(0.1, 60, 90, "step", 0, 10) == pytest.approx(0.1 * 0.01)
    assert lr_policy.learning_rate(0.1, 45, 90, "polynomial", 0, 10) == pytest.approx(0.025)
    assert lr_policy.learning_rate(0.1, 2, 90, "step", 9, 10, lr_warmup=True) == pytest.approx(0.1 * 30 / 50)
    with pytest.raises(NotImplementedError):
        lr_policy.learning_rate(0.1, 0, 90, "cosine", 0, 10)


class _FakeRuntime(object):
    def __init__(self, stage, ranks, first):
        self.stage, self.num_ranks_in_stage, self.num_ranks_in_first_stage = stage, ranks, first

    def get_adjusted_learning_rate(self, base_lr):   # runtime/runtime.py:673-680
        if self.stage == 0:
            return base_lr
        return float(base_lr) * float(self.num_ranks_in_stage) / float(self.num_ranks_in_first_stage)


class _FakeOptimizer(object):
    def __init__(self):
        self.param_groups = [{"lr": 1.0}, {"lr": 2.0}]


def test_adjust_writes_every_param_group_and_scales_by_replicas():
    opt = _FakeOptimizer()
    r = _FakeRuntime(stage=2, ranks=1, first=4)
    lr = lr_policy.adjust_learning_rate(opt, 30, 90, r, "step", 5, 100, base_lr=0.4)
    assert lr == pytest.approx(0.4 / 4 * 0.1)
    assert [g["lr"] for g in opt.param_groups] == [lr, lr]
    sched = lr_policy.schedule_for(r, 0.4, 1, 90, "step", 100, lr_warmup=True)
    assert sched(49) == pytest.approx(0.1 * 150 / 500)
