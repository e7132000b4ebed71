"""Writes tests/golden/mlp_c1.json: losses and parameter checksums of the small
CPU-runnable configuration (2-stage MLP 784-1024-1024-10, batch 64, SGD lr 0.01
momentum 0.9 wd 1e-4, 2 weight versions on stage 0, 20 minibatches, seed 0) computed by
the CPU oracle (oracle/pipeline_oracle.py on torch.nn modules).  Nothing from the
reference tree is imported or run.

Usage: python tests/golden/make_mlp_golden.py
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import models, pipeline_oracle, stash_oracle  # noqa: E402


def make_batches(n=20, batch=64, d_in=784, classes=10, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(batch, d_in, generator=g), torch.randint(0, classes, (batch,), generator=g))
            for _ in range(n)]


def make_stages(seed=0):
    torch.manual_seed(seed)
    return [models.MlpStage0(), models.MlpStage1()]


SGD_KW = dict(lr=0.01, momentum=0.9, weight_decay=1e-4)


def run():
    stages = make_stages()
    batches = make_batches()
    losses, st = pipeline_oracle.run_pipeline(
        stages, torch.nn.CrossEntropyLoss(),
        lambda s, m, nv: stash_oracle.StashingOptimizerOracle("SGD", [m], m.parameters(), nv, **SGD_KW),
        batches)
    params = {}
    for s, m in enumerate(stages):
        for k, v in m.state_dict().items():
            v = v.double()
            params["stage%d.%s" % (s, k)] = {"sum": float(v.sum()), "abs_sum": float(v.abs().sum()),
                                             "first": [float(x) for x in v.flatten()[:4]]}
    return {"config": "mlp 784-1024-1024-10, bs64, SGD lr .01 mom .9 wd 1e-4, versions 2/1, 20 steps, seed 0",
            "losses": losses, "params": params,
            "fwd_versions": [x.fwd_versions for x in st], "bwd_versions": [x.bwd_versions for x in st]}


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mlp_c1.json")
    with open(out, "w") as f:
        json.dump(run(), f, indent=1)
    print("wrote", out)
