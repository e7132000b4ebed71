"""VGG16 stages on the HIP kernels against the CPU oracle (torch.nn twins in
oracle/models.py, weight stashing restated in oracle/stash_oracle.py).

* the conv1_1..pool2 stage of the headline configuration at reduced size: per-minibatch
  outputs, input-side versions and parameters after a stash-depth-4 1F1B run;
* the full 4-stage VGG16 pipeline (stash depths 4/3/2/1, device-buffer hand-off, injected
  dropout masks) at batch 2: losses, versions, parameters;
* at the full benchmark size (batch 64, 224x224): size-independent properties --
  exact homogeneity under power-of-two scaling and the adjoint identities
  <conv(x,w),dy> = <x,dgrad(dy,w)> = <w,wgrad(x,dy)> that tie the three kernels together.

Tolerance: rel 1e-5 on losses; parameters rtol 1e-5 with atol 1e-6 (a few ulp at the
parameters' magnitude)."""
import copy

import pytest
import torch

from oracle import models
from oracle import stash_oracle as so

pytestmark = pytest.mark.gpu

SGD_KW = dict(lr=0.01, momentum=0.9, weight_decay=5e-4)


def _nhwc(t):
    return t.cuda().contiguous(memory_format=torch.channels_last)


def test_front_stage_1f1b_matches_oracle():
    from pipedream_amd import sgd
    from pipedream_amd.stages import vgg16
    torch.manual_seed(0)
    ref = models.VggFrontStage()
    mine = vgg16.FrontStage()
    mine.load_state_dict(ref.state_dict())       # reference-format checkpoint loads as is
    mine = mine.cuda()
    W, nv, n = 3, 4, 8
    opt = sgd.SGDWithWeightStashing([mine], list(mine.parameters()), None, 1.0, nv, **SGD_KW)
    ora = so.StashingOptimizerOracle("SGD", [ref], ref.parameters(), nv, **SGD_KW)
    g = torch.Generator().manual_seed(1)
    xs = [torch.randn(2, 3, 32, 32, generator=g) for _ in range(n)]
    gs = [torch.randn(2, 128, 8, 8, generator=g) * 1e-3 for _ in range(n)]
    pend_ref, pend = [], []
    for kind, k in so.one_f_one_b(n, W):
        if kind == "F":
            assert opt.latest_version.version == so.forward_version(k, W)
            yr = ref(xs[k])
            y = mine(_nhwc(xs[k]))
            torch.testing.assert_close(y.cpu(), yr.detach(), rtol=1e-5, atol=1e-5)
            pend_ref.append(yr)
            pend.append(y)
        else:
            for o in (ora, opt):
                o.zero_grad()
                o.load_old_params()
            assert opt.current_version.version == ora.current_version == so.backward_version(k, W)
            pend_ref.pop(0).backward(gs[k])
            pend.pop(0).backward(_nhwc(gs[k]))
            for o in (ora, opt):
                o.load_new_params()
                o.step()
            assert opt.queue.versions() == ora.versions()
    got = mine.state_dict()
    for key, v in ref.state_dict().items():
        torch.testing.assert_close(got[key].cpu(), v, rtol=1e-5, atol=1e-6)
        assert got[key].shape == v.shape


def _load(name):
    import importlib.util
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    spec = importlib.util.spec_from_file_location(name, os.path.join(here, "golden", name + ".py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod, here


def test_full_vgg16_four_stage_pipeline_matches_oracle():
    """4 co-resident stages, stash depths 4/3/2/1, batch 2, 5 minibatches.

    Versions are bit-exact.  Minibatches 0 and 1 (a pure forward, then one update of the
    last stage) must match to rel 1e-5.  Beyond that the reference path itself is only
    reproducible to the committed noise floor (tests/golden/vgg16_noise_floor.json: the
    CPU oracle in fp32 against itself in fp64, see make_vgg_noise_floor.py for why); the
    product has to stay within a small multiple of that floor of the fp32 oracle."""
    import json
    import os
    from pipedream_amd import handoff, runtime, schedule, sgd
    from pipedream_amd.layers import CrossEntropyLoss
    from pipedream_amd.stages import vgg16
    nf, here = _load("make_vgg_noise_floor")
    floor = json.load(open(os.path.join(here, "golden", "vgg16_noise_floor.json")))
    n, batch = nf.N_MINIBATCHES, nf.BATCH

    ref_losses, ref_stages, ref_st = nf.run_oracle(torch.float32)

    masks = nf.dropout_masks()
    count = {"layer13": 0, "layer16": 0}
    handoff.reset_fabrics()
    model = vgg16.model(CrossEntropyLoss(), dropout=0.5)
    fresh = nf.make_stages(None)                       # same seed -> the oracle's initial weights
    for (m, _, _), ref in zip(model[:4], fresh):
        m.load_state_dict(ref.state_dict())
    for name in ("layer13", "layer16"):
        def mask_fn(x, name=name):
            i = count[name]
            count[name] += 1
            return masks[name][i].to(torch.uint8).cuda()
        getattr(model[3][0], name).mask_fn = mask_fn

    conf = vgg16.conf()
    shapes = {"input0": (batch, 3, 224, 224), "target": (batch,)}
    dtypes = {"input0": torch.float32, "target": torch.int64}
    stages = []
    for rank in range(4):
        r = runtime.StageRuntime(
            model=model, distributed_backend="gloo", fp16=False, loss_scale=1.0,
            training_tensor_shapes=shapes, eval_tensor_shapes=dict(shapes), training_tensor_dtypes=dtypes,
            inputs_module_destinations={"input": 0}, target_tensor_names={"target"},
            configuration_maps={"module_to_stage_map": conf["module_to_stage_map"],
                                "stage_to_rank_map": conf["stage_to_rank_map"], "stage_to_depth_map": None},
            master_addr="127.0.0.1", rank=rank, local_rank=0, num_ranks_in_server=4, verbose_freq=0,
            model_type=runtime.IMAGE_CLASSIFICATION)
        opt = sgd.SGDWithWeightStashing(r.modules(), r.master_parameters, r.model_parameters, 1.0,
                                        num_versions=r.num_warmup_minibatches + 1, **SGD_KW)
        stages.append((r, opt))
    assert [r.num_warmup_minibatches for r, _ in stages] == [3, 2, 1, 0]     # stash depths 4/3/2/1
    assert [o.num_versions for _, o in stages] == [4, 3, 2, 1]

    batches = nf.make_batches()
    losses = []
    loops = [schedule.stage_train_loop(
        r, o, n, loader=batches if i == 0 else None,
        on_forward=(lambda k, rr: losses.append(float(rr.loss.detach()))) if i == 3 else None)
        for i, (r, o) in enumerate(stages)]
    schedule.run_pipeline(loops)
    torch.cuda.synchronize()

    assert [st.optimizer.versions() for st in ref_st] == [o.queue.versions() for _, o in stages]
    # The floor is ONE realisation of a noise process that grows ~100x per minibatch once the
    # first ReLU / pooling decision has flipped, and which minibatch that happens in is a
    # matter of chance; so from minibatch 2 on a run may be one minibatch "ahead" of the
    # recorded realisation.
    fl = floor["loss_rel"]
    for k, (a, b) in enumerate(zip(losses, ref_losses)):
        ahead = fl[min(k + 1, len(fl) - 1)] if k >= 2 else fl[k]
        tol = max(1e-5, 3 * ahead * (3 if k == len(fl) - 1 else 1))
        assert abs(a - b) <= tol * abs(b) + 1e-6, (k, losses, ref_losses)
    assert fl[0] < 1e-5 and fl[1] < 1e-5
    for si, ((r, _), ref) in enumerate(zip(stages, ref_stages)):
        got = r.modules()[0].state_dict()
        for key, v in ref.state_dict().items():
            err = float((got[key].cpu() - v).norm() / v.norm())
            tol = max(1e-5, 10 * floor["param_rel_l2"]["stage%d.%s" % (si, key)])
            assert err <= tol, (si, key, err, tol)


@pytest.fixture(params=["direct", "winograd"])
def conv_algorithm(request):
    from pipedream_amd import ops
    ops.set_conv_algorithm(request.param)
    yield request.param
    ops.set_conv_algorithm("auto")


def test_full_size_conv_properties(conv_algorithm):
    """Batch 64, 224x224, 64 -> 64 channels (the heaviest layer of the benchmark stage), under the direct and
    the Winograd kernels: size-independent identities instead of an oracle run."""
    from pipedream_amd import ops
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(64, 64, 224, 224, device="cuda", generator=gen).contiguous(memory_format=torch.channels_last)
    w = (torch.randn(64, 64, 3, 3, device="cuda", generator=gen) / 24).contiguous(memory_format=torch.channels_last)
    y = ops.conv3x3_forward(x, w)
    # homogeneity: scaling an operand by a power of two scales the result exactly
    assert torch.equal(ops.conv3x3_forward(x * 2, w), y * 2)
    assert torch.equal(ops.conv3x3_forward(x, w * 0.5), y * 0.5)
    dy = torch.randn(64, 64, 224, 224, device="cuda", generator=gen).contiguous(memory_format=torch.channels_last)
    dx = ops.conv3x3_input_grad(dy, w)
    dw, db = ops.conv3x3_weight_grad(x, dy)
    # adjoint identities (fp64 reductions of fp32 products)
    lhs = (y.double() * dy.double()).sum()
    via_dx = (x.double() * dx.double()).sum()
    via_dw = (w.double() * dw.double()).sum()
    scale = (y.double().abs() * dy.double().abs()).sum()
    assert abs(lhs - via_dx) <= 1e-6 * scale, (float(lhs), float(via_dx))
    assert abs(lhs - via_dw) <= 1e-6 * scale, (float(lhs), float(via_dw))
    # bias gradient is the plain sum over pixels
    ref_db = dy.double().sum(dim=(0, 2, 3))
    torch.testing.assert_close(db.double(), ref_db, rtol=1e-5, atol=1e-5 * float(dy.double().abs().sum() / 64) ** 0.5)
    # a constant-one 3x3 filter on one channel counts neighbours: interior 9, edges 6, corners 4
    ones = torch.ones(1, 4, 8, 8, device="cuda").contiguous(memory_format=torch.channels_last)
    k = torch.zeros(4, 4, 3, 3, device="cuda")
    k[0, 0] = 1
    cnt = ops.conv3x3_forward(ones, k.contiguous(memory_format=torch.channels_last))[0, 0]
    assert cnt[0, 0] == 4 and cnt[0, 3] == 6 and cnt[3, 3] == 9 and cnt[7, 7] == 4
    if conv_algorithm == "winograd":
        # the two algorithms agree to fp32 rounding at full size (outputs are O(1): 576-term sums of N(0,1)/24)
        del dx, dw
        ops.set_conv_algorithm("direct")
        y_direct = ops.conv3x3_forward(x, w)
        assert float((y - y_direct).abs().max()) < 2e-5
        dw_w, _ = (ops.set_conv_algorithm("winograd"), ops.conv3x3_weight_grad(x, dy))[1]
        dw_d, _ = (ops.set_conv_algorithm("direct"), ops.conv3x3_weight_grad(x, dy))[1]
        assert float((dw_w - dw_d).abs().max()) <= 1e-5 * float(dw_d.abs().max())
