"""Pins of the two oracle pieces that check the bf16 pre-LN transformer stage.  CPU only.

The reference checkout holds no transformer stage and no 2BW optimizer (README.md:7-8 sends
the reader to another branch), so there is no reference file or vector to match: **parity
unpinned by reference, pinned on the library** --

(i)   ``oracle.models.TransformerLayerOracle`` composes attention by hand (split, reshape,
      scale, softmax).  With its products and LayerNorms evaluated in fp32 it must equal
      ``torch.nn.TransformerEncoderLayer(norm_first=True, activation='gelu', dropout=0)``
      carrying the same weights, output and every gradient, to 1e-6.
(ii)  Its bf16 evaluation (what the HIP tests compare with) stays within 2e-2 rel-L2 of (i).
(iii) Mutants of the oracle's source (softmax scale 1/d, post-LN, q and k exchanged with v in
      the split, tanh GELU, heads split before the q/k/v split) each fail (i).
(iv)  ``StashingOptimizerOracle(update_interval=4, num_versions=2)`` with Adam equals "sum four
      gradients, divide by four, ``torch.optim.Adam.step``" written out by hand, over 12
      micro-batches, and its ring holds versions [j-1, j] after update j."""
import inspect
import textwrap

import pytest
import torch

from oracle import models as om, stash_oracle as so

H, HEADS, FFN = 32, 4, 64


class _Fp32Layer(om.TransformerLayerOracle):
    """The oracle's forward, unchanged, with the two precision hooks evaluated in fp32."""

    @staticmethod
    def _lin(x, m):
        return torch.nn.functional.linear(x, m.weight, m.bias)

    @staticmethod
    def _ln(x, m):
        return torch.nn.functional.layer_norm(x, x.shape[-1:], m.weight, m.bias, m.eps)


def _library_twin(layer):
    lib = torch.nn.TransformerEncoderLayer(H, HEADS, FFN, dropout=0.0, activation='gelu',
                                           batch_first=True, norm_first=True)
    with torch.no_grad():
        lib.self_attn.in_proj_weight.copy_(layer.qkv.weight)
        lib.self_attn.in_proj_bias.copy_(layer.qkv.bias)
        lib.self_attn.out_proj.weight.copy_(layer.proj.weight)
        lib.self_attn.out_proj.bias.copy_(layer.proj.bias)
        lib.linear1.weight.copy_(layer.fc1.weight)
        lib.linear1.bias.copy_(layer.fc1.bias)
        lib.linear2.weight.copy_(layer.fc2.weight)
        lib.linear2.bias.copy_(layer.fc2.bias)
        for a, b in ((lib.norm1, layer.ln1), (lib.norm2, layer.ln2)):
            a.weight.copy_(b.weight)
            a.bias.copy_(b.bias)
    lib.train()      # the inference fast path of the library layer is a different kernel; stay on the plain one
    return lib


_PAIRS = [("qkv.weight", "self_attn.in_proj_weight"), ("qkv.bias", "self_attn.in_proj_bias"),
          ("proj.weight", "self_attn.out_proj.weight"), ("proj.bias", "self_attn.out_proj.bias"),
          ("fc1.weight", "linear1.weight"), ("fc1.bias", "linear1.bias"),
          ("fc2.weight", "linear2.weight"), ("fc2.bias", "linear2.bias"),
          ("ln1.weight", "norm1.weight"), ("ln1.bias", "norm1.bias"),
          ("ln2.weight", "norm2.weight"), ("ln2.bias", "norm2.bias")]


def _make(cls, seed=0):
    torch.manual_seed(seed)
    layer = cls(H, HEADS, FFN)
    with torch.no_grad():   # LayerNorm's default weight 1 / bias 0 would hide a mistake in their use
        for ln in (layer.ln1, layer.ln2):
            ln.weight.add_(0.3 * torch.randn(H))
            ln.bias.add_(0.3 * torch.randn(H))
    return layer


def _inputs(seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(3, 10, H, generator=g), torch.randn(3, 10, H, generator=g)


def _compare_with_library(cls, tol=1e-6):
    layer = _make(cls)
    lib = _library_twin(layer)
    x, dy = _inputs()
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya, yb = layer(xa), lib(xb)
    ya.backward(dy)
    yb.backward(dy)
    worst = float((ya.detach() - yb.detach()).abs().max() / yb.detach().abs().max())
    worst = max(worst, float((xa.grad - xb.grad).abs().max() / xb.grad.abs().max()))
    pa, pb = dict(layer.named_parameters()), dict(lib.named_parameters())
    for na, nb in _PAIRS:
        if pa[na].grad is None:       # a parameter the (mutated) forward never used
            return float("inf"), tol
        worst = max(worst, float((pa[na].grad - pb[nb].grad).abs().max() / pb[nb].grad.abs().max()))
    return worst, tol


def test_fp32_evaluation_equals_library_encoder_layer():
    worst, tol = _compare_with_library(_Fp32Layer)
    assert worst <= tol, worst


def test_bf16_evaluation_stays_within_tolerance_of_fp32():
    ref, low = _make(_Fp32Layer), _make(om.TransformerLayerOracle)
    x, dy = _inputs()
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya = ref(xa)
    yb = low(xb.bfloat16())
    assert yb.dtype == torch.bfloat16
    ya.backward(dy)
    yb.backward(dy.bfloat16())

    def rel(a, b):
        return float((a.float() - b.float()).norm() / b.float().norm())
    assert rel(yb, ya) <= 2e-2
    assert rel(xb.grad, xa.grad) <= 2e-2
    for (n, pa), (_, pb) in zip(ref.named_parameters(), low.named_parameters()):
        assert pb.grad.dtype == torch.float32 and rel(pb.grad, pa.grad) <= 2e-2, n


_MUTANTS = [
    ("(1.0 / d ** 0.5)", "(1.0 / d)"),                                              # softmax scale
    ("x = self._lin(att, self.proj) + x", "x = self._ln(self._lin(att, self.proj) + x, self.ln1)"),   # post-LN
    ("q, k, v = [", "v, k, q = ["),                                                 # roles in the packed projection
    ("torch.nn.functional.gelu(self._lin(self._ln(x, self.ln2), self.fc1))",
     "torch.nn.functional.gelu(self._lin(self._ln(x, self.ln2), self.fc1), approximate='tanh')"),
    ("p = torch.softmax((q @ k.transpose(-1, -2))", "p = torch.softmax((k @ q.transpose(-1, -2))"),   # transposed scores
    ("self._ln(x, self.ln2)", "self._ln(x, self.ln1)"),                             # wrong LayerNorm in the MLP branch
    ("return self._lin(f, self.fc2) + x", "return self._lin(f, self.fc2)"),         # dropped residual
    ("[t.reshape(B, S, self.heads, d).transpose(1, 2) for t in qkv.split(H, dim=-1)]",
     "[t.reshape(B, S, d, self.heads).permute(0, 3, 1, 2) for t in qkv.split(H, dim=-1)]"),          # head-minor split
]


@pytest.mark.parametrize("old,new", _MUTANTS)
def test_mutants_of_the_oracle_fail_the_library_pin(old, new):
    src = textwrap.dedent(inspect.getsource(om.TransformerLayerOracle.forward))
    assert src.count(old) == 1, "the mutation site moved: " + old
    ns = {"torch": torch}
    exec(compile(src.replace(old, new), "<mutant>", "exec"), ns)
    mutant = type("Mutant", (_Fp32Layer,), {"forward": ns["forward"]})
    worst, tol = _compare_with_library(mutant)
    assert worst > 100 * tol, (old, worst)


def test_decoupled_interval_adam_equals_accumulate_average_then_library_step():
    """update_interval=4 with num_versions=2 (the 2BW arrangement): gradients of four micro-batches are summed,
    divided by four and applied once; the ring then holds the previous and the new version."""
    kw = dict(lr=1e-2, betas=(0.9, 0.99), weight_decay=1e-3)

    def make():
        torch.manual_seed(3)
        return torch.nn.Sequential(torch.nn.Linear(6, 5), torch.nn.Tanh(), torch.nn.Linear(5, 3))
    a, b = make(), make()
    opt = so.StashingOptimizerOracle("Adam", [a], a.parameters(), 2, update_interval=4, **kw)
    assert opt.num_versions == 2 and opt.update_interval == 4
    ref = torch.optim.Adam(b.parameters(), **kw)
    g = torch.Generator().manual_seed(4)
    xs = [torch.randn(7, 6, generator=g) for _ in range(12)]
    for i in range(0, 12, 4):
        sums = [torch.zeros_like(p) for p in b.parameters()]
        for x in xs[i:i + 4]:
            grads = torch.autograd.grad(b(x).pow(2).mean(), list(b.parameters()))
            sums = [s + gr for s, gr in zip(sums, grads)]
        for p, s in zip(b.parameters(), sums):
            p.grad = s / 4
        ref.step()
    for i, x in enumerate(xs):
        opt.zero_grad()
        opt.load_new_params()       # all four micro-batches of an interval run on the newest weights
        a(x).pow(2).mean().backward()
        opt.step()
        done = (i + 1) // 4
        assert opt.versions() == ([0, 0] if done == 0 else [done - 1, done])
    for pa, pb in zip(a.parameters(), b.parameters()):
        torch.testing.assert_close(pa, pb, rtol=1e-6, atol=1e-7)
    # the older slot still holds the weights before the last update: one more hand-rolled check
    opt.load_old_params()
    assert not any(torch.equal(pa, pb) for pa, pb in zip(a.parameters(), b.parameters()))
    opt.load_new_params()
    for pa, pb in zip(a.parameters(), b.parameters()):
        torch.testing.assert_close(pa, pb, rtol=1e-6, atol=1e-7)
