"""The small CPU-runnable configuration end to end: 2-stage MLP 784-1024-1024-10, batch
64, SGDWithWeightStashing lr 0.01 momentum 0.9 wd 1e-4, 2 versions on stage 0, 20
minibatches, seed 0.

CPU part: the oracle reproduces the committed golden vectors.  GPU part: two co-resident
``StageRuntime``s + ``SGDWithWeightStashing`` (HIP kernels, device-buffer hand-off)
against the golden vectors and against a live oracle run: version selection bit-exact,
losses and parameters within rel 1e-5 (fp32 tolerance of the north-star)."""
import importlib.util
import json
import os

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_mlp_golden", os.path.join(HERE, "golden", "make_mlp_golden.py"))
gold = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(gold)

GOLDEN = json.load(open(os.path.join(HERE, "golden", "mlp_c1.json")))
RTOL = 1e-5


def test_oracle_reproduces_golden():
    got = gold.run()
    assert got["fwd_versions"] == GOLDEN["fwd_versions"]
    assert got["bwd_versions"] == GOLDEN["bwd_versions"]
    for a, b in zip(got["losses"], GOLDEN["losses"]):
        assert abs(a - b) <= RTOL * abs(b) + 1e-6
    for k, v in GOLDEN["params"].items():
        assert abs(got["params"][k]["abs_sum"] - v["abs_sum"]) <= RTOL * v["abs_sum"]


def test_golden_versions_follow_the_closed_form():
    from oracle import stash_oracle as so
    assert GOLDEN["fwd_versions"][0] == [so.forward_version(k, 1) for k in range(20)]
    assert GOLDEN["bwd_versions"][0] == [so.backward_version(k, 1) for k in range(20)]
    assert GOLDEN["fwd_versions"][1] == list(range(20)) == GOLDEN["bwd_versions"][1]


def _build_product(num_minibatches=20):
    from pipedream_amd import handoff, runtime, sgd
    from pipedream_amd.layers import CrossEntropyLoss
    from pipedream_amd.stages import mlp

    handoff.reset_fabrics()
    torch.manual_seed(0)
    model = mlp.model(CrossEntropyLoss())
    conf = mlp.conf()
    shapes = {"input0": (64, 784), "target": (64,), "out0": (64, 1024), "out1": (64, 10)}
    dtypes = {"input0": torch.float32, "target": torch.int64, "out0": torch.float32, "out1": torch.float32}
    stages = []
    for rank in range(2):
        r = runtime.StageRuntime(
            model=model, distributed_backend="gloo", fp16=False, loss_scale=1.0,
            training_tensor_shapes=shapes, eval_tensor_shapes=dict(shapes), training_tensor_dtypes=dtypes,
            inputs_module_destinations={"input": 0}, target_tensor_names={"target"},
            configuration_maps={"module_to_stage_map": conf["module_to_stage_map"],
                                "stage_to_rank_map": conf["stage_to_rank_map"], "stage_to_depth_map": None},
            master_addr="127.0.0.1", rank=rank, local_rank=0, num_ranks_in_server=2, verbose_freq=0,
            model_type=runtime.IMAGE_CLASSIFICATION)
        opt = sgd.SGDWithWeightStashing(r.modules(), r.master_parameters, r.model_parameters, 1.0,
                                        num_versions=r.num_warmup_minibatches + 1, **gold.SGD_KW)
        stages.append((r, opt))
    return stages


def _run_product(n, per_stage_streams=False, minibatch_rings=False):
    """n minibatches through the two co-resident stages.  Returns losses, the version every
    forward/backward ran on, the final state_dicts and the ReLU masks of every forward."""
    from pipedream_amd import schedule
    stages = _build_product()
    # no host synchronisation around the run: the loops order their streams against the caller's themselves
    streams = schedule.stage_streams(len(stages)) if per_stage_streams else [None] * len(stages)
    assert [r.num_warmup_minibatches for r, _ in stages] == [1, 0]
    assert [o.num_versions for _, o in stages] == [2, 1]
    batches = gold.make_batches()[:n]
    losses, masks = [], []
    versions = [{"F": [], "B": []} for _ in stages]
    s0 = stages[0][0].modules()[0]
    for layer in (s0.layer1, s0.layer2):      # fused Linear+ReLU: output > 0 is the mask
        layer.register_forward_hook(lambda m, i, o: masks.append((o.detach() > 0).cpu()))
    loops = []
    for si, (r, opt) in enumerate(stages):
        orig_fwd, orig_bwd = r.run_forward, r.run_backward

        def fwd(orig=orig_fwd, si=si, opt=opt):
            versions[si]["F"].append(opt.latest_version.version)
            orig()

        def bwd(orig=orig_bwd, si=si, opt=opt):
            versions[si]["B"].append(opt.current_version.version if opt.num_versions > 1
                                     else opt.latest_version.version)
            orig()

        r.run_forward, r.run_backward = fwd, bwd
        loops.append(schedule.stage_train_loop(
            r, opt, n, loader=batches if si == 0 else None,
            on_forward=(lambda i, rr: losses.append(float(rr.loss.detach()))) if si == 1 else None,
            stream=streams[si],
            minibatch_streams=schedule.MinibatchStreams(r.num_warmup_minibatches) if minibatch_rings else None))
    schedule.run_pipeline(loops)
    params = [{k: v.detach().cpu() for k, v in r.modules()[0].state_dict().items()} for r, _ in stages]
    return losses, versions, params, masks


def _run_oracle(n):
    from oracle import pipeline_oracle, stash_oracle
    ref_stages = gold.make_stages()
    masks = []
    for layer in (ref_stages[0].layer1, ref_stages[0].layer2):
        layer.register_forward_hook(lambda m, i, o: masks.append(o.detach() > 0))
    losses, _ = pipeline_oracle.run_pipeline(
        ref_stages, torch.nn.CrossEntropyLoss(),
        lambda s, m, nv: stash_oracle.StashingOptimizerOracle("SGD", [m], m.parameters(), nv, **gold.SGD_KW),
        gold.make_batches()[:n])
    return losses, [dict(m.state_dict()) for m in ref_stages], masks


def _assert_params_close(mine, ref):
    for got, want in zip(mine, ref):
        for k, v in want.items():
            torch.testing.assert_close(got[k], v, rtol=RTOL, atol=1e-6)


@pytest.mark.gpu
def test_product_matches_golden_and_oracle():
    n = 20
    losses, versions, params, masks = _run_product(n)
    # bit-exact version selection
    assert [v["F"] for v in versions] == GOLDEN["fwd_versions"]
    assert [v["B"] for v in versions] == GOLDEN["bwd_versions"]
    # every loss within rel 1e-5 of the golden vector
    for a, b in zip(losses, GOLDEN["losses"]):
        assert abs(a - b) <= RTOL * abs(b) + 1e-6, (losses, GOLDEN["losses"])

    # Parameters against a live oracle run, full tensors.  ReLU's derivative is
    # discontinuous: when a pre-activation is within fp32 rounding of zero, two correct
    # fp32 implementations that sum in a different order can take different sides, and
    # from that minibatch on their parameters differ by far more than rounding.  Such
    # events are detected by comparing the masks of the two runs; parameters must agree
    # elementwise (rel 1e-5) over the longest prefix of minibatches free of such a flip,
    # and stay within 1e-2 in relative L2 norm beyond it.
    ref_losses, ref_params, ref_masks = _run_oracle(n)
    assert len(masks) == len(ref_masks) == 2 * n
    flipped = [i // 2 for i, (a, b) in enumerate(zip(masks, ref_masks)) if not torch.equal(a, b)]
    first_flip = min(flipped) if flipped else None
    if first_flip is None:
        _assert_params_close(params, ref_params)
    else:
        assert first_flip >= 8, "mask flips this early point at an error, not at rounding"
        for got, want in zip(params, ref_params):
            for k, v in want.items():
                assert float((got[k] - v).norm() / v.norm()) < 1e-2
        _, _, p_prefix, m_prefix = _run_product(first_flip)
        _, ref_prefix, ref_m_prefix = _run_oracle(first_flip)
        assert all(torch.equal(a, b) for a, b in zip(m_prefix, ref_m_prefix))
        _assert_params_close(p_prefix, ref_prefix)
    for si in range(2):
        for k, v in params[si].items():
            gv = GOLDEN["params"]["stage%d.%s" % (si, k)]
            assert abs(float(v.double().abs().sum()) - gv["abs_sum"]) <= 1e-4 * gv["abs_sum"] + 1e-6


@pytest.mark.gpu
def test_one_stream_per_stage_gives_the_same_bits():
    """Each stage launching on a stream of its own, ordered by the hand-off's events: the same kernels on the
    same operands in an order that respects every dependency, so losses, versions, masks and parameters
    are identical, bit for bit, to the single-stream run."""
    n = 12
    one = _run_product(n)
    many = _run_product(n, per_stage_streams=True)
    assert one[0] == many[0] and one[1] == many[1]
    for a, b in zip(one[2], many[2]):
        assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)
    assert all(torch.equal(a, b) for a, b in zip(one[3], many[3]))


@pytest.mark.gpu
def test_minibatch_stream_rings_give_the_same_bits():
    """Every stage with a ``MinibatchStreams`` ring (forward of a new minibatch beside the backward of the oldest
    in flight), the stages ordered by the hand-off's events: identical to the single-stream run, bit for bit."""
    n = 12
    one = _run_product(n)
    many = _run_product(n, minibatch_rings=True)
    assert one[0] == many[0] and one[1] == many[1]
    for a, b in zip(one[2], many[2]):
        assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)
    assert all(torch.equal(a, b) for a, b in zip(one[3], many[3]))


@pytest.mark.gpu
def test_schedule_detects_deadlock():
    from pipedream_amd import schedule
    stages = _build_product()
    r1, o1 = stages[1]
    # only the last stage runs: it can never receive its input
    with pytest.raises(RuntimeError, match="deadlocked"):
        schedule.run_pipeline([schedule.stage_train_loop(r1, o1, 2)])
