"""Host logic of ``StageRuntime``: the static wiring of a stage (which tensors enter and leave it, who
sends them, warm-up depths) against the reference's rules (runtime/runtime.py:162-175, :192-222) on
hand-worked layouts, and the hand-off queue contract.  No GPU needed."""
import pytest
import torch

from pipedream_amd import handoff
from pipedream_amd.runtime import _StageWiring


def _model(spec):
    return [(object(), ins, outs) for ins, outs in spec]


STRAIGHT4 = _model([(["input0"], ["out0"]), (["out0"], ["out1"]), (["out1"], ["out2"]), (["out2"], ["out3"]),
                    (["out3"], ["loss"])])


def _wire(model, m2s, s2r, rank, depth=None, dest=None, targets=("target",)):
    return _StageWiring(model, m2s, s2r, depth, dest or {"input": 0}, set(targets), rank)


def test_straight_four_stage_pipeline():
    s2r = {"0": [0], "1": [1], "2": [2], "3": [3]}
    ws = [_wire(STRAIGHT4, [0, 1, 2, 3, 3], s2r, r) for r in range(4)]
    assert [w.warmup for w in ws] == [3, 2, 1, 0]
    assert [w.has_criterion for w in ws] == [False, False, False, True]
    assert [w.entries for w in ws] == [("input0",), ("out0",), ("out1",), ("out2",)]
    assert [w.exits for w in ws] == [("out0",), ("out1",), ("out2",), ("loss",)]
    assert [w.returned for w in ws] == [(), ("out0",), ("out1",), ("out2",)]
    assert ws[0].inbound == {} and ws[0].outbound == {"out0": 1, "target": 1}
    assert ws[2].inbound == {"out1": 1, "target": 1} and ws[2].outbound == {"out2": 3, "target": 3}
    assert ws[3].inbound == {"out2": 2, "target": 2} and ws[3].outbound == {}
    assert all(w.num_stages == 4 and w.num_ranks == 4 for w in ws)


def test_depth_map_overrides_and_single_stage():
    s2r = {0: [0], 1: [1]}
    w = _wire(STRAIGHT4, [0, 0, 1, 1, 1], s2r, 0, depth={"0": 5, "1": 0})
    assert w.warmup == 5 and w.entries == ("input0",) and w.exits == ("out1",)
    one = _wire(STRAIGHT4, None, None, None)
    assert one.stage is None and one.warmup == 0 and one.has_criterion
    assert one.entries == ("input0",) and one.exits == ("loss",) and not one.inbound and not one.outbound


def test_forwarded_model_input():
    """A model input whose destination module sits in stage 1 travels there from stage 0, next to the
    activation (runtime/runtime.py:208-222); only the activation's gradient goes back."""
    model = _model([(["input0"], ["out0"]), (["out0", "input1"], ["out1"]), (["out1"], ["out2"]),
                    (["out2"], ["loss"])])
    s2r = {0: [0], 1: [1], 2: [2]}
    dest = {"input0": 0, "input1": 1}
    w0 = _wire(model, [0, 1, 2, 2], s2r, 0, dest=dest)
    w1 = _wire(model, [0, 1, 2, 2], s2r, 1, dest=dest)
    assert w0.outbound == {"out0": 1, "input1": 1, "target": 1}
    assert w1.inbound == {"out0": 0, "input1": 0, "target": 0}
    assert w1.entries == ("out0", "input1") and w1.returned == ("out0",)


def test_replicated_stage_is_refused():
    with pytest.raises(NotImplementedError, match="replicated"):
        _wire(STRAIGHT4, [0, 0, 1, 1, 1], {0: [0, 1], 1: [2]}, 0)


def test_handoff_queue_contract():
    handoff.reset_fabrics()
    a = handoff.DeviceHandoff("k", 0, {}, {"out0": 1})
    b = handoff.DeviceHandoff("k", 1, {"out0": 0}, {}, ack_to=0)
    x = torch.ones(3, requires_grad=True) * 2
    ids = torch.arange(3)
    assert not b.ready(["out0"], backward=False)
    a.put("out0", x, 0, backward=False, premasked=True)
    a.put("out0", ids, 1, backward=False)
    assert b.ready(["out0"], backward=False)
    p = b.take("out0", 0, backward=False)
    # detached from the sender's graph, a gradient-requiring leaf on receipt (communication.py:595-596, :699)
    assert p.tensor.is_leaf and p.tensor.requires_grad and p.premasked and p.tensor.data_ptr() == x.data_ptr()
    q = b.take("out0", 1, backward=False)
    assert not q.tensor.requires_grad and not q.premasked          # integer tensors stay as they are
    with pytest.raises(RuntimeError, match="nothing queued"):
        b.take("out0", 2, backward=False)
    # gradients go back along the same route, in order
    b.put("out0", torch.zeros(3), 0, backward=True)
    b.put("out0", torch.zeros(3), 1, backward=True)
    a.take("out0", 0, backward=True)
    with pytest.raises(RuntimeError, match="arrived where"):
        a.take("out0", 5, backward=True)
    # a new run drops stale backward traffic addressed to the stage, keeps forward traffic
    b.put("out0", torch.zeros(3), 2, backward=True)
    a.put("out0", x, 0, backward=False)
    a.begin_run(forward_only=True)
    b.begin_run(forward_only=True)
    assert not a.ready(["out0"], backward=True) and b.ready(["out0"], backward=False)
