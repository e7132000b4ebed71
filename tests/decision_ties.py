"""Test helper: the ReLU / max-pooling decisions of a CPU oracle stage, and the oracle re-run with chosen
decisions switched.

ReLU and max-pooling are not differentiable where a pre-activation is zero or two candidates of a window
are equal.  Two correct fp32 evaluations of the same stage (another summation order) agree on the
activations to ~1e-6 relative, so among the millions of decisions of a VGG stage at 224x224 now and then
one operand lies closer to its kink than that, the two evaluations take different branches, and the
gradients they return differ by the whole contribution of that element.  Neither is wrong: each is the
exact gradient for an input moved by less than the rounding of the forward pass.

``Decisions`` records, during a forward pass of the oracle module, the input of every ``relu`` /
``max_pool2d`` call and can list the decisions with the smallest margins; run again with ``switch=[...]``
it adds to those inputs a nudge of a few times the margin (well below 1e-5 of the activations' scale) that
makes the listed decisions go the other way, everything else being untouched.  A parity test can then state
a tie precisely: the product equals the oracle evaluated on activations moved by less than the tolerance.
"""
import collections

import torch
from torch.overrides import TorchFunctionMode

Tie = collections.namedtuple("Tie", "call kind index margin scale nudge_at nudge")


class Decisions(TorchFunctionMode):
    def __init__(self, switch=()):
        super(Decisions, self).__init__()
        self.inputs = []                    # (kind, detached input) per call, in call order
        self._switch = collections.defaultdict(list)
        for t in switch:
            self._switch[t.call].append(t)

    def __torch_function__(self, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        name = getattr(func, "__name__", "")
        if name in ("relu", "max_pool2d") and args and torch.is_tensor(args[0]) and args[0].dim() >= 2:
            x = args[0]
            call = len(self.inputs)
            self.inputs.append((name, x.detach()))
            if call in self._switch:
                bump = torch.zeros_like(x.detach())
                for t in self._switch[call]:
                    bump.view(-1)[t.nudge_at] += t.nudge
                x = x + bump
            return func(x, *args[1:], **kwargs)      # runs below this mode: nested calls are not recorded
        return func(*args, **kwargs)

    def closest(self, count=16):
        """The ``count`` decisions with the smallest margins relative to their tensor's scale."""
        out = []
        for call, (kind, x) in enumerate(self.inputs):
            scale = float(x.std())
            flat = x.reshape(-1)
            if kind == "relu":
                margin = flat.abs()
                k = min(count, margin.numel())
                vals, idx = torch.topk(margin, k, largest=False)
                for m, i in zip(vals.tolist(), idx.tolist()):
                    z = float(flat[i])
                    # push the pre-activation across zero by twice its distance (at least a few ulp of the scale)
                    step = 2 * abs(z) + 4e-7 * scale
                    out.append(Tie(call, kind, i, m / scale, scale, i, -step if z > 0 else step))
            else:
                n, c, h, w = x.shape
                win = x[:, :, :h // 2 * 2, :w // 2 * 2].reshape(n, c, h // 2, 2, w // 2, 2).permute(0, 1, 2, 4, 3, 5)
                win = win.reshape(n, c, h // 2, w // 2, 4)
                top = torch.topk(win, 2, dim=-1)
                gap = (top.values[..., 0] - top.values[..., 1]).reshape(-1)
                # windows of a rectified tensor that hold nothing positive tie at zero exactly; whichever
                # element the gradient is routed to, the ReLU before the pooling sets it to zero
                gap = torch.where(top.values[..., 0].reshape(-1) > 0, gap, torch.full_like(gap, float("inf")))
                k = min(count, gap.numel())
                vals, idx = torch.topk(gap, k, largest=False)
                # the candidate the pooling does not take: the runner-up, or for two equal values the later one
                # in scan order (max_pool2d keeps the first maximum it meets)
                first, second = top.indices[..., 0].reshape(-1), top.indices[..., 1].reshape(-1)
                second = torch.where(gap == 0, torch.maximum(first, second), second)
                for g, i in zip(vals.tolist(), idx.tolist()):
                    ww = i % (w // 2)
                    hh = (i // (w // 2)) % (h // 2)
                    nc = i // ((w // 2) * (h // 2))
                    j = int(second[i])
                    at = (nc * h + hh * 2 + j // 2) * w + ww * 2 + j % 2
                    out.append(Tie(call, kind, i, g / scale, scale, at, 2 * g + 4e-7 * scale))
        out.sort(key=lambda t: t.margin)
        return out[:count]


def stage_backward(module, x, grad_out, target=None, criterion=None, switch=()):
    """Forward + backward of an oracle stage module on ``x`` (a leaf is made of it) with the decisions in
    ``switch`` taken the other way.  Returns (output, input gradient or None, {parameter name: gradient},
    the Decisions record)."""
    for p in module.parameters():
        p.grad = None
    x = x.detach().clone()
    if x.dtype.is_floating_point:
        x.requires_grad_()
    rec = Decisions(switch)
    with rec:
        out = module(x)
        if criterion is not None:
            out = criterion(out, target)
    if criterion is not None:
        out.backward()
    else:
        torch.autograd.backward((out,), grad_tensors=(grad_out,))
    grads = {n: p.grad.detach().clone() for n, p in module.named_parameters()}
    return out.detach(), (x.grad if x.requires_grad else None), grads, rec
