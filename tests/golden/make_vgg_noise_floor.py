"""Writes tests/golden/vgg16_noise_floor.json: how far the CPU oracle's fp32 trajectory of
the 4-stage VGG16 pipeline (batch 2, 5 minibatches, stash depths 4/3/2/1, SGD lr 0.01
momentum 0.9 wd 5e-4, injected dropout masks) lies from the same oracle run in fp64.

Why: ReLU and max-pooling are not differentiable where a pre-activation is zero / two
window candidates are equal.  With ~3e7 such decisions per minibatch some operands lie
within fp32 rounding of the kink, and any two correct fp32 evaluations (different
summation order, or fp32 vs fp64) take different branches there.  At batch 2 each such
decision moves a gradient by ~1e-3 relative and the optimizer compounds it, so the
trajectory of the *reference path itself* is only reproducible to the figures recorded
here.  The GPU parity test holds the product to a small multiple of this floor (and to
rel 1e-5 where the floor is below that).

Nothing from the reference tree is imported or run.  Usage:
    python tests/golden/make_vgg_noise_floor.py      (about a minute on 8 cores)
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import models, pipeline_oracle  # noqa: E402
from oracle import stash_oracle as so  # noqa: E402

SGD_KW = dict(lr=0.01, momentum=0.9, weight_decay=5e-4)
N_MINIBATCHES, BATCH = 5, 2


def dropout_masks(seed=5):
    g = torch.Generator().manual_seed(seed)
    return {name: [(torch.rand(BATCH, 4096, generator=g) >= 0.5) for _ in range(N_MINIBATCHES)]
            for name in ("layer13", "layer16")}


def make_batches(seed=2):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(BATCH, 3, 224, 224, generator=g), torch.randint(0, 1000, (BATCH,), generator=g))
            for _ in range(N_MINIBATCHES)]


def make_stages(mask_fn, seed=0):
    torch.manual_seed(seed)
    return [models.VggStage0(), models.VggStage1(), models.VggStage2(),
            models.VggStage3(dropout=0.5, masks=mask_fn)]


def run_oracle(dtype=torch.float32, observer=None):
    masks = dropout_masks()
    count = {"layer13": 0, "layer16": 0}

    def mask_fn(name, x):
        i = count[name]
        count[name] += 1
        return masks[name][i]

    stages = [s.to(dtype) for s in make_stages(mask_fn)]
    batches = [(x.to(dtype), t) for x, t in make_batches()]
    old = pipeline_oracle.LEAF_DTYPES
    pipeline_oracle.LEAF_DTYPES = (torch.float32, torch.float64)
    try:
        losses, st = pipeline_oracle.run_pipeline(
            stages, torch.nn.CrossEntropyLoss(),
            lambda s, m, nv: so.StashingOptimizerOracle("SGD", [m], m.parameters(), nv, **SGD_KW), batches,
            observer=observer)
    finally:
        pipeline_oracle.LEAF_DTYPES = old
    return losses, stages, st


if __name__ == "__main__":
    l32, s32, _ = run_oracle(torch.float32)
    l64, s64, _ = run_oracle(torch.float64)
    out = {"config": "VGG16 4 stages, batch 2, 5 minibatches, SGD lr .01 mom .9 wd 5e-4, seeds 0/2/5",
           "loss_rel": [abs(a - b) / abs(b) for a, b in zip(l32, l64)], "param_rel_l2": {}}
    for i, (a, b) in enumerate(zip(s32, s64)):
        sb = b.state_dict()
        for k, v in a.state_dict().items():
            out["param_rel_l2"]["stage%d.%s" % (i, k)] = float((v.double() - sb[k]).norm() / sb[k].norm())
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vgg16_noise_floor.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)
