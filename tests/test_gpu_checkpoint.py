"""Checkpoint / resume in the reference's format
(runtime/image_classification/main_with_runtime.py:319-330 save, :211-218 and :232 resume):
per stage ``{'state_dict': r.state_dict(), 'optimizer': optimizer.state_dict()}`` where
``r.state_dict()`` is ``{"module%d": module.state_dict()}`` (runtime/runtime.py:306-321) and
the optimizer entry is the *base* optimizer's state dict; the version ring is not saved and
is re-seeded with identical clones on resume (runtime/optimizer.py:58-62).

The product is run 6 minibatches, checkpointed through ``torch.save``, rebuilt, resumed and
run 4 more; the CPU oracle does the same with ``torch.nn`` / ``torch.optim``.  Parameters
must agree to rel 1e-5, and each side's checkpoint must load into the other."""
import copy
import io

import pytest
import torch

import test_pipeline_mlp as T

pytestmark = pytest.mark.gpu
gold = T.gold


def _product_segment(batches, ckpt=None):
    from pipedream_amd import handoff, runtime, schedule, sgd
    from pipedream_amd.layers import CrossEntropyLoss
    from pipedream_amd.stages import mlp
    handoff.reset_fabrics()
    torch.manual_seed(123)                       # different init: resume must overwrite it
    model = mlp.model(CrossEntropyLoss())
    if ckpt is None:
        torch.manual_seed(0)
        model = mlp.model(CrossEntropyLoss())
    conf = mlp.conf()
    shapes = {"input0": (64, 784), "target": (64,)}
    dtypes = {"input0": torch.float32, "target": torch.int64}
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
        if ckpt is not None:
            r.load_state_dict(ckpt[rank]["state_dict"])          # before the optimizer exists
        opt = sgd.SGDWithWeightStashing(r.modules(), r.master_parameters, r.model_parameters, 1.0,
                                        num_versions=r.num_warmup_minibatches + 1, **gold.SGD_KW)
        if ckpt is not None:
            opt.load_state_dict(ckpt[rank]["optimizer"])
        stages.append((r, opt))
    loops = [schedule.stage_train_loop(r, o, len(batches), loader=batches if i == 0 else None)
             for i, (r, o) in enumerate(stages)]
    schedule.run_pipeline(loops)
    torch.cuda.synchronize()
    buf = io.BytesIO()
    torch.save([{"state_dict": r.state_dict(), "optimizer": o.state_dict()} for r, o in stages], buf)
    buf.seek(0)
    return stages, torch.load(buf, map_location="cpu", weights_only=True)


def _oracle_segment(batches, ckpt=None):
    from oracle import pipeline_oracle, stash_oracle
    ref = gold.make_stages(seed=0 if ckpt is None else 123)
    if ckpt is not None:
        for m, c in zip(ref, ckpt):
            m.load_state_dict(c["state_dict"]["module0"])
    opts = {}

    def make(s, m, nv):
        o = stash_oracle.StashingOptimizerOracle("SGD", [m], m.parameters(), nv, **gold.SGD_KW)
        if ckpt is not None:
            o.base_optimizer.load_state_dict(ckpt[s]["optimizer"])
        opts[s] = o
        return o

    pipeline_oracle.run_pipeline(ref, torch.nn.CrossEntropyLoss(), make, batches)
    out = []
    for s, m in enumerate(ref):
        sd = {"module0": m.state_dict()}
        if s == len(ref) - 1:
            sd["module1"] = torch.nn.CrossEntropyLoss().state_dict()   # the criterion is the stage's last module
        out.append({"state_dict": sd, "optimizer": opts[s].base_optimizer.state_dict()})
    return ref, out


def test_checkpoint_resume_matches_oracle_and_formats_interchange():
    batches = gold.make_batches()
    first, second = batches[:6], batches[6:10]
    _, ck_mine = _product_segment(first)
    _, ck_ref = _oracle_segment(first)

    # same format: keys, shapes, optimizer layout
    for a, b in zip(ck_mine, ck_ref):
        assert list(a["state_dict"].keys()) == list(b["state_dict"].keys())   # module0 (+ criterion)
        assert list(a["state_dict"]["module0"].keys()) == list(b["state_dict"]["module0"].keys())
        for k, v in b["state_dict"]["module0"].items():
            assert a["state_dict"]["module0"][k].shape == v.shape
            torch.testing.assert_close(a["state_dict"]["module0"][k], v, rtol=1e-5, atol=1e-6)
        assert a["optimizer"]["param_groups"][0]["momentum"] == b["optimizer"]["param_groups"][0]["momentum"]
        assert set(a["optimizer"]["state"].keys()) == set(b["optimizer"]["state"].keys())
        for i, st in b["optimizer"]["state"].items():
            torch.testing.assert_close(a["optimizer"]["state"][i]["momentum_buffer"], st["momentum_buffer"],
                                       rtol=1e-5, atol=1e-6)

    # resume each side from its own checkpoint
    st_mine, _ = _product_segment(second, ck_mine)
    # torch's load_state_dict aliases same-device state tensors, so hand each consumer its own copy
    ref, _ = _oracle_segment(second, copy.deepcopy(ck_ref))
    for (r, _), m in zip(st_mine, ref):
        got = r.modules()[0].state_dict()
        for k, v in m.state_dict().items():
            torch.testing.assert_close(got[k].cpu(), v, rtol=1e-5, atol=1e-6)

    # cross-load: the product resumes from the oracle's (reference-format) checkpoint
    st_cross, _ = _product_segment(second, ck_ref)
    for (r, _), m in zip(st_cross, ref):
        got = r.modules()[0].state_dict()
        for k, v in m.state_dict().items():
            torch.testing.assert_close(got[k].cpu(), v, rtol=1e-5, atol=1e-6)
    # after a resume the ring holds identical clones at version 0 + the new updates
    assert st_mine[0][1].queue.versions() == [3, 4]


def test_checkpoint_holds_one_copy_of_every_tensor():
    """The live parameters are views into the version ring and the momentum buffers views into one flat
    buffer; what ``state_dict()`` hands to ``torch.save`` must not drag the ring's other slots along: the file
    is about the size of the parameters plus the optimizer state."""
    stages, _ = _product_segment(gold.make_batches()[:3])
    buf = io.BytesIO()
    torch.save([{"state_dict": r.state_dict(), "optimizer": o.state_dict()} for r, o in stages], buf)
    n_params = sum(p.numel() for r, _ in stages for p in r.parameters())
    assert stages[0][1].num_versions == 2                       # a ring with more than one slot is in play
    expected = 2 * 4 * n_params                                 # parameters + momentum, fp32
    assert expected <= buf.getbuffer().nbytes <= 1.02 * expected + (1 << 16)
