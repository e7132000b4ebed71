"""The weight-gradient entry point that allocates nothing (pd_conv3x3_wgrad_noalloc_nhwc_f32) against
pd_conv3x3_wgrad_nhwc_f32 with a caller's workspace: the same kernels on the library's built-in scratch
array, so the results must agree bit for bit -- on two calls in a row, the second with a smaller input
(the array keeps the first call's partial sums), for the few-channel and the 64-channel kernels, with and
without the ReLU mask.  A shape beyond the array is refused."""
import ctypes
import gc

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else None)


def _both(lib, N, H, W, C, K, masked, seed):
    from pipedream_amd import _cabi
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(N, H, W, C, device="cuda", generator=g)
    dy = torch.randn(N, H, W, K, device="cuda", generator=g)
    mask = torch.relu(torch.randn(N, H, W, K, device="cuda", generator=g)) if masked else None
    need = ctypes.c_uint64()
    lib.pd_conv3x3_wgrad_workspace_bytes(N, H, W, C, K, ctypes.byref(need))
    ws = torch.empty(need.value, dtype=torch.uint8, device="cuda")
    out = []
    for which in ("workspace", "noalloc"):
        dw = torch.full((K, 3, 3, C), float("nan"), device="cuda")
        db = torch.full((K,), float("nan"), device="cuda")
        stream = _cabi.stream_ptr()
        if which == "workspace":
            lib.pd_conv3x3_wgrad_nhwc_f32(_ptr(x), _ptr(dy), _ptr(mask), _ptr(dw), _ptr(db), _ptr(ws), need.value,
                                          N, H, W, C, K, stream)
        else:
            if not _both.warm:
                # the first call on a device resolves the scratch array's address and is not measured
                lib.pd_conv3x3_wgrad_noalloc_nhwc_f32(_ptr(x), _ptr(dy), _ptr(mask), _ptr(dw), _ptr(db),
                                                      N, H, W, C, K, stream)
                _both.warm = True
            gc.collect()
            torch.cuda.synchronize()
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            lib.pd_conv3x3_wgrad_noalloc_nhwc_f32(_ptr(x), _ptr(dy), _ptr(mask), _ptr(dw), _ptr(db),
                                                  N, H, W, C, K, stream)
            torch.cuda.synchronize()
            # nothing was taken from torch's allocator, nothing from the device (a hipMalloc inside the library
            # would show there); either figure may still fall when frees that earlier tests left pending complete
            assert torch.cuda.memory_allocated() <= before
            assert torch.cuda.mem_get_info()[0] >= free_before
        out.append((dw, db))
    torch.cuda.synchronize()
    return x, dy, mask, out, need.value


_both.warm = False


@pytest.mark.parametrize("C,K,first,second", [(3, 64, (4, 64, 64), (1, 17, 9)),      # few-channel kernel
                                              (64, 64, (2, 40, 40), (1, 8, 8)),      # pipelined kernel
                                              (20, 12, (2, 19, 23), (1, 5, 7))])     # scalar kernel, ragged sizes
@pytest.mark.parametrize("masked", [False, True])
def test_two_calls_in_a_row_match_the_workspace_entry_point(C, K, first, second, masked):
    from pipedream_amd import _cabi
    lib = _cabi.lib()
    for seed, (N, H, W) in enumerate((first, second)):
        x, dy, mask, ((dw_a, db_a), (dw_b, db_b)), need = _both(lib, N, H, W, C, K, masked, seed)
        assert need <= 16 << 20
        assert torch.equal(dw_a, dw_b) and torch.equal(db_a, db_b)
        assert not torch.isnan(dw_b).any() and not torch.isnan(db_b).any()
        # and both are the weight gradient: fp64 conv2d weight gradient on the CPU
        xr = x.permute(0, 3, 1, 2).double().cpu()
        g = dy if mask is None else dy * (mask > 0)
        gr = g.permute(0, 3, 1, 2).double().cpu()
        w = torch.zeros(K, C, 3, 3, dtype=torch.float64, requires_grad=True)
        torch.nn.functional.conv2d(xr, w, padding=1).backward(gr)
        ref = w.grad.permute(0, 2, 3, 1)
        assert float((dw_b.double().cpu() - ref).norm() / ref.norm()) <= 1e-5
        ref_b = gr.sum(dim=(0, 2, 3))
        assert float((db_b.double().cpu() - ref_b).norm() / ref_b.norm()) <= 1e-5


def test_full_size_first_layer_fits_and_matches():
    """conv1_1 of the benchmark stage (batch 64, 224x224, 3 -> 64 channels) fits the scratch array."""
    from pipedream_amd import _cabi
    lib = _cabi.lib()
    _, _, _, ((dw_a, db_a), (dw_b, db_b)), need = _both(lib, 64, 224, 224, 3, 64, False, 5)
    assert need <= 16 << 20
    assert torch.equal(dw_a, dw_b) and torch.equal(db_a, db_b)


def test_shape_beyond_the_scratch_array_is_refused():
    from pipedream_amd import _cabi
    lib = _cabi.lib()
    N, H, W, C, K = 64, 112, 112, 128, 128
    need = ctypes.c_uint64()
    lib.pd_conv3x3_wgrad_workspace_bytes(N, H, W, C, K, ctypes.byref(need))
    assert need.value > 16 << 20
    x = torch.zeros(16, device="cuda")
    with pytest.raises(_cabi.PipedreamAmdError, match="scratch array holds") as e:
        # refused on the sizes alone, before any pointer is used
        lib.pd_conv3x3_wgrad_noalloc_nhwc_f32(_ptr(x), _ptr(x), None, _ptr(x), None, N, H, W, C, K,
                                              _cabi.stream_ptr())
    assert e.value.code == -2
