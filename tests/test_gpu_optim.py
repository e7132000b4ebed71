"""Parity of the fused optimizer kernels (through the C ABI) with the CPU oracle.

Tolerance: fp32, rel 1e-5 (+ atol 5e-7, a few ulp of the O(1) operands, for entries that cancel to ~0), the bar the
north-star sets for parameters after N steps."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import stash_oracle as so
from pipedream_amd import _cabi

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 5e-7


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _desc_array(entries):
    arr = (_cabi.TensorDesc * len(entries))()
    for d, e in zip(arr, entries):
        d.grad, d.p_in, d.p_out = e["g"].data_ptr(), e["p_in"].data_ptr(), e["p_out"].data_ptr()
        d.state0 = e["s0"].data_ptr() if e.get("s0") is not None else None
        d.state1 = e["s1"].data_ptr() if e.get("s1") is not None else None
        d.bf16_out = e["bf16"].data_ptr() if e.get("bf16") is not None else None
        d.n = e["p_in"].numel()
    return arr


SIZES = [1, 3, 4, 63, 64, 257, 4096, 4097, 100003, 1 << 20]


@pytest.mark.parametrize("momentum,dampening,wd,nesterov", [
    (0.0, 0.0, 0.0, False), (0.9, 0.0, 5e-4, False), (0.9, 0.1, 1e-4, False), (0.9, 0.0, 1e-4, True)])
def test_sgd_multi_tensor_vs_oracle(momentum, dampening, wd, nesterov):
    lib = _cabi.lib()
    rng = np.random.RandomState(0)
    ps = [rng.randn(n).astype(np.float32) for n in SIZES]
    bufs = [None] * len(SIZES)
    d_p = [_dev(p) for p in ps]
    d_out = [torch.empty_like(t) for t in d_p]
    d_buf = [torch.zeros_like(t) for t in d_p]
    for step in range(4):
        gs = [rng.randn(n).astype(np.float32) for n in SIZES]
        d_g = [_dev(g) for g in gs]
        entries = [dict(g=g, p_in=p, p_out=o, s0=b if momentum else None)
                   for g, p, o, b in zip(d_g, d_p, d_out, d_buf)]
        lib.pd_sgd_step(_desc_array(entries), len(entries), 0.05, momentum, dampening, wd, int(nesterov),
                        int(step == 0), 1.0, 1.0, _cabi.stream_ptr())
        torch.cuda.synchronize()
        for i in range(len(SIZES)):
            ps[i], bufs[i] = so.sgd_step_numpy(ps[i], gs[i], bufs[i], 0.05, momentum, dampening, wd, nesterov)
            np.testing.assert_allclose(d_out[i].cpu().numpy(), ps[i], rtol=RTOL, atol=ATOL)
            if momentum:
                np.testing.assert_allclose(d_buf[i].cpu().numpy(), bufs[i], rtol=RTOL, atol=ATOL)
        d_p, d_out = d_out, d_p   # out-of-place ping-pong, like two ring slots


@pytest.mark.parametrize("eps_mode,wd", [(0, 0.0), (0, 1e-2), (1, 0.0)])
def test_adam_multi_tensor_vs_oracle(eps_mode, wd):
    lib = _cabi.lib()
    rng = np.random.RandomState(1)
    ps = [rng.randn(n).astype(np.float32) for n in SIZES]
    ms = [np.zeros(n, np.float32) for n in SIZES]
    vs = [np.zeros(n, np.float32) for n in SIZES]
    d_p = [_dev(p) for p in ps]
    d_m = [torch.zeros_like(t) for t in d_p]
    d_v = [torch.zeros_like(t) for t in d_p]
    d_h = [torch.zeros(t.numel(), dtype=torch.bfloat16, device="cuda") for t in d_p]
    for step in range(1, 5):
        gs = [rng.randn(n).astype(np.float32) for n in SIZES]
        d_g = [_dev(g) for g in gs]
        entries = [dict(g=g, p_in=p, p_out=p, s0=m, s1=v, bf16=h)
                   for g, p, m, v, h in zip(d_g, d_p, d_m, d_v, d_h)]
        lib.pd_adam_step(_desc_array(entries), len(entries), 1e-3, 0.9, 0.999, 1e-8, wd, step, eps_mode, 1.0, 1.0,
                         _cabi.stream_ptr())
        torch.cuda.synchronize()
        for i in range(len(SIZES)):
            ps[i], ms[i], vs[i] = so.adam_step_numpy(ps[i], gs[i], ms[i], vs[i], step, 1e-3, 0.9, 0.999, 1e-8, wd,
                                                     eps_mode)
            np.testing.assert_allclose(d_p[i].cpu().numpy(), ps[i], rtol=RTOL, atol=ATOL)
            np.testing.assert_allclose(d_m[i].cpu().numpy(), ms[i], rtol=RTOL, atol=ATOL)
            np.testing.assert_allclose(d_v[i].cpu().numpy(), vs[i], rtol=RTOL, atol=1e-9)
            # bf16 image = round-to-nearest-even of the fp32 result
            assert torch.equal(d_h[i], d_p[i].to(torch.bfloat16))


_TORCH16 = {"bf16": torch.bfloat16, "f16": torch.float16}


@pytest.mark.parametrize("grad_fmt,out_fmt", [("f32", "f16"), ("f32", "bf16"), ("bf16", "bf16"), ("f16", "f16"),
                                              ("bf16", "f16"), ("f16", "bf16")])
@pytest.mark.parametrize("adam", [False, True])
def test_mixed_step_every_format_pair_vs_oracle(grad_fmt, out_fmt, adam):
    """Every (gradient format, 16-bit copy format) pair the header allows for pd_*_step_mixed, aligned and
    ragged sizes: the fp32 results equal the oracle's step on the widened gradient, the 16-bit copy is the
    rounded fp32 result bit for bit.  (fp32 gradients with an fp16 copy once read the gradients as 16-bit.)"""
    lib = _cabi.lib()
    code = {"f32": _cabi.PD_F32, "bf16": _cabi.PD_BF16, "f16": _cabi.PD_F16}
    rng = np.random.RandomState(5)
    sizes = [5, 4096, 4097, 100003]
    ps = [rng.randn(n).astype(np.float32) for n in sizes]
    ms = [np.zeros(n, np.float32) for n in sizes]
    vs = [np.zeros(n, np.float32) for n in sizes]
    bufs = [None] * len(sizes)
    d_p = [_dev(p) for p in ps]
    d_m = [torch.zeros_like(t) for t in d_p]
    d_v = [torch.zeros_like(t) for t in d_p]
    d_h = [torch.zeros(t.numel(), dtype=_TORCH16[out_fmt], device="cuda") for t in d_p]
    for step in range(1, 4):
        gs = [rng.randn(n).astype(np.float32) for n in sizes]
        d_g = [_dev(g) for g in gs]
        if grad_fmt != "f32":
            d_g = [g.to(_TORCH16[grad_fmt]) for g in d_g]
            gs = [g.float().cpu().numpy() for g in d_g]
        entries = [dict(g=g, p_in=p, p_out=p, s0=m, s1=v if adam else None, bf16=h)
                   for g, p, m, v, h in zip(d_g, d_p, d_m, d_v, d_h)]
        if adam:
            lib.pd_adam_step_mixed(_desc_array(entries), len(entries), 1e-3, 0.9, 0.999, 1e-8, 1e-2, step, 0, 1.0, 1.0,
                                   code[grad_fmt], code[out_fmt], _cabi.stream_ptr())
        else:
            lib.pd_sgd_step_mixed(_desc_array(entries), len(entries), 0.05, 0.9, 0.0, 1e-4, 0, int(step == 1), 1.0,
                                  1.0, code[grad_fmt], code[out_fmt], _cabi.stream_ptr())
        torch.cuda.synchronize()
        for i in range(len(sizes)):
            if adam:
                ps[i], ms[i], vs[i] = so.adam_step_numpy(ps[i], gs[i], ms[i], vs[i], step, 1e-3, 0.9, 0.999, 1e-8, 1e-2, 0)
                np.testing.assert_allclose(d_v[i].cpu().numpy(), vs[i], rtol=RTOL, atol=1e-9)
                np.testing.assert_allclose(d_m[i].cpu().numpy(), ms[i], rtol=RTOL, atol=ATOL)
            else:
                ps[i], bufs[i] = so.sgd_step_numpy(ps[i], gs[i], bufs[i], 0.05, 0.9, 0.0, 1e-4, False)
                np.testing.assert_allclose(d_m[i].cpu().numpy(), bufs[i], rtol=RTOL, atol=ATOL)
            np.testing.assert_allclose(d_p[i].cpu().numpy(), ps[i], rtol=RTOL, atol=ATOL)
            assert torch.equal(d_h[i], d_p[i].to(_TORCH16[out_fmt]))


def test_unaligned_views_take_the_scalar_path():
    lib = _cabi.lib()
    rng = np.random.RandomState(2)
    n = 5000
    base = [_dev(rng.randn(n + 3).astype(np.float32)) for _ in range(3)]
    g, p, b = [t[1:1 + n] for t in base]      # 4-byte aligned only
    g0, p0 = g.cpu().numpy().copy(), p.cpu().numpy().copy()
    lib.pd_sgd_step(_desc_array([dict(g=g, p_in=p, p_out=p, s0=b)]), 1, 0.1, 0.9, 0.0, 0.0, 0, 1, 1.0, 1.0,
                    _cabi.stream_ptr())
    want, buf = so.sgd_step_numpy(p0, g0, None, 0.1, 0.9)
    np.testing.assert_allclose(p.cpu().numpy(), want, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(b.cpu().numpy(), buf, rtol=RTOL, atol=ATOL)
    # neighbours untouched
    assert base[1][0].item() == base[1][0].item() and torch.isfinite(base[1]).all()


def test_grad_scaling_is_a_true_division():
    lib = _cabi.lib()
    rng = np.random.RandomState(3)
    g, p = rng.randn(9999).astype(np.float32), rng.randn(9999).astype(np.float32)
    dg, dp = _dev(g), _dev(p)
    lib.pd_sgd_step(_desc_array([dict(g=dg, p_in=dp, p_out=dp)]), 1, 0.5, 0.0, 0.0, 0.0, 0, 0, 128.0, 3.0,
                    _cabi.stream_ptr())
    want, _ = so.sgd_step_numpy(p, (g / np.float32(128.0)) / np.float32(3.0), None, 0.5)
    np.testing.assert_allclose(dp.cpu().numpy(), want, rtol=RTOL, atol=ATOL)


def test_more_tensors_than_one_launch_holds():
    lib = _cabi.lib()
    rng = np.random.RandomState(4)
    sizes = [17 + 5 * i for i in range(75)] + [0, 9000]
    ps = [rng.randn(n).astype(np.float32) for n in sizes]
    gs = [rng.randn(n).astype(np.float32) for n in sizes]
    d_p, d_g = [_dev(p) for p in ps], [_dev(g) for g in gs]
    lib.pd_sgd_step(_desc_array([dict(g=g, p_in=p, p_out=p) for g, p in zip(d_g, d_p)]), len(sizes), 0.1, 0.0, 0.0,
                    0.0, 0, 0, 1.0, 1.0, _cabi.stream_ptr())
    for p, g, dp in zip(ps, gs, d_p):
        np.testing.assert_allclose(dp.cpu().numpy(), so.sgd_step_numpy(p, g, None, 0.1)[0], rtol=RTOL, atol=ATOL)


def test_full_size_linearity_property():
    """VGG16-sized flat buffer (138 357 544 parameters): with momentum 0 and wd 0 the step is
    p' = p - lr*g exactly in fp32 when lr is a power of two, a size-independent check that
    every element was visited exactly once."""
    lib = _cabi.lib()
    n = 138357544
    gen = torch.Generator(device="cuda").manual_seed(0)
    p = torch.randn(n, device="cuda", generator=gen)
    g = torch.randn(n, device="cuda", generator=gen)
    out = torch.full((n + 64,), 7.0, device="cuda")
    lib.pd_sgd_step(_desc_array([dict(g=g, p_in=p, p_out=out[:n])]), 1, 0.5, 0.0, 0.0, 0.0, 0, 0, 1.0, 1.0,
                    _cabi.stream_ptr())
    assert torch.equal(out[:n], p - 0.5 * g)
    assert (out[n:] == 7.0).all()


def test_copy_fill_and_ring_broadcast():
    lib = _cabi.lib()
    for n in (4, 12, 1000, 1 << 20, (1 << 20) + 12):
        src = torch.randn(n // 4, device="cuda")
        dst = torch.zeros_like(src)
        lib.pd_copy(ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()), n, _cabi.stream_ptr())
        assert torch.equal(src, dst)
        lib.pd_fill_zero(ctypes.c_void_p(dst.data_ptr()), n, _cabi.stream_ptr())
        assert not dst.any()
    stride = 1 << 16
    buf = torch.randn(3 * stride // 4, device="cuda")
    h = ctypes.c_void_p()
    lib.pd_ring_create(ctypes.c_void_p(buf.data_ptr()), stride, 3, ctypes.byref(h))
    lib.pd_ring_broadcast(h, 2, stride, _cabi.stream_ptr())
    v = buf.view(3, -1)
    assert torch.equal(v[0], v[2]) and torch.equal(v[1], v[2])
    lib.pd_ring_destroy(h)
