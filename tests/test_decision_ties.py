"""The tie helper of the VGG parity test (tests/decision_ties.py) on a case worked by hand: it finds the
decision that lies at its kink, and switching it moves the gradient from one branch to the other while the
forward result moves by less than 1e-5."""
import torch

import decision_ties as dt


class _Tiny(torch.nn.Module):
    def __init__(self):
        super(_Tiny, self).__init__()
        self.scale = torch.nn.Parameter(torch.ones(1))

    def forward(self, x):
        return torch.nn.functional.max_pool2d(torch.relu(x * self.scale), 2, 2)


def _input():
    x = torch.tensor([[1.0, 2.0, -3.0, 5.0],
                      [2.0 - 2e-7, 0.5, 4.0, -1.0],
                      [3e-8, -2.0, 7.0, 7.0],
                      [-1.0, -4.0, 1.0, 2.0]]).reshape(1, 1, 4, 4)
    return x


def test_closest_decisions_are_the_near_ties():
    m = _Tiny()
    out, gx, grads, rec = dt.stage_backward(m, _input(), torch.ones(1, 1, 2, 2))
    assert [k for k, _ in rec.inputs] == ["relu", "max_pool2d"]
    ties = rec.closest(4)
    found = {(t.kind, t.nudge_at) for t in ties}
    # 7 == 7 in the last window (the later one in scan order is not taken), 2 vs 2 - 2e-7 in the first, the 3e-8
    # ReLU, and the window whose only positive entry is that 3e-8 (its runner-up is a rectified zero)
    assert found >= {("max_pool2d", 11), ("max_pool2d", 4), ("relu", 8)}
    assert len(found) == 4 and (found - {("max_pool2d", 11), ("max_pool2d", 4), ("relu", 8)}).pop()[1] in (9, 12, 13)
    assert ties[0].margin == 0.0


def test_switching_one_decision_moves_its_gradient_only():
    m = _Tiny()
    x = _input()
    out0, g0, _, rec = dt.stage_backward(m, x, torch.ones(1, 1, 2, 2))
    assert g0.reshape(-1).tolist() == [0, 1, 0, 1, 0, 0, 0, 0, 1, 0, 1, 0, 0, 0, 0, 0]
    by_place = {(t.kind, t.nudge_at): t for t in rec.closest(4)}
    # pooling tie of window 0: the gradient moves from x[0,1] to x[1,0]
    out1, g1, _, _ = dt.stage_backward(m, x, torch.ones(1, 1, 2, 2), switch=[by_place["max_pool2d", 4]])
    assert g1.reshape(-1).tolist() == [0, 0, 0, 1, 1, 0, 0, 0, 1, 0, 1, 0, 0, 0, 0, 0]
    # exact tie of window 3: from the first 7 to the second
    out2, g2, _, _ = dt.stage_backward(m, x, torch.ones(1, 1, 2, 2), switch=[by_place["max_pool2d", 11]])
    assert g2.reshape(-1).tolist() == [0, 1, 0, 1, 0, 0, 0, 0, 1, 0, 0, 1, 0, 0, 0, 0]
    # the ReLU at 3e-8 switched off: window 2 holds nothing positive any more, its gradient is masked
    out3, g3, _, _ = dt.stage_backward(m, x, torch.ones(1, 1, 2, 2), switch=[by_place["relu", 8]])
    assert g3.reshape(-1).tolist() == [0, 1, 0, 1, 0, 0, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0]
    scale = float(x.std())
    for o in (out1, out2, out3):
        assert float((o - out0).abs().max()) <= 1e-5 * scale
    # two at once
    _, g4, _, _ = dt.stage_backward(m, x, torch.ones(1, 1, 2, 2),
                                    switch=[by_place["max_pool2d", 4], by_place["max_pool2d", 11]])
    assert g4.reshape(-1).tolist() == [0, 0, 0, 1, 1, 0, 0, 0, 1, 0, 0, 1, 0, 0, 0, 0]
