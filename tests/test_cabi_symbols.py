"""The C-ABI library loads without a GPU and exports exactly what include/*.h declares."""
import ctypes
import os
import re
import subprocess

import pytest

from pipedream_amd import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pipedream_amd.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(pd_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared() == sorted(_cabi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    dll = ctypes.CDLL(_cabi.LIB_PATH)
    for name in _declared():
        assert hasattr(dll, name), "libpipedream_amd.so does not export %s" % name


def test_no_undeclared_exports():
    out = subprocess.run(["nm", "-D", "--defined-only", _cabi.LIB_PATH], capture_output=True, text=True).stdout
    exported = set(re.findall(r"\bT (pd_[a-z0-9_]+)$", out, flags=re.M))
    assert exported - {"pd_set_error"} <= set(_declared()), exported - set(_declared())


def test_abi_version_and_error_string():
    lib = _cabi.lib()
    assert lib.pd_abi_version() == 1
    with pytest.raises(_cabi.PipedreamAmdError) as ei:
        lib.pd_copy(None, None, 16, None)
    assert "NULL" in str(ei.value)
    # argument validation happens on the host before any launch
    with pytest.raises(_cabi.PipedreamAmdError):
        lib.pd_copy(ctypes.c_void_p(4096), ctypes.c_void_p(8192), 6, None)
    with pytest.raises(_cabi.PipedreamAmdError):
        lib.pd_adam_step(None, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0, 0, 1.0, 1.0, None)


def test_product_refuses_cpu_tensors():
    import torch
    from pipedream_amd import sgd
    if torch.cuda.is_available():
        pytest.skip("host-only check")
    model = torch.nn.Linear(4, 4)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        sgd.SGDWithWeightStashing([model], list(model.parameters()), None, 1.0, 2, lr=0.1)


def test_convolution_algorithm_choice_is_host_logic():
    """Which kernel a 3x3 convolution takes is decided on the host from shapes alone: Winograd for channel
    counts it supports and that pay, the direct kernels otherwise -- including images the Winograd kernels
    cannot address with 32-bit offsets."""
    from pipedream_amd import ops
    assert ops._use_winograd(64, 64, 224, 224)
    assert ops._use_winograd(128, 128, 112, 112)
    assert not ops._use_winograd(3, 64, 224, 224)          # few channels: the dense-tap kernels
    assert not ops._use_winograd(20, 70, 17, 33)           # K % 4 != 0
    assert not ops._use_winograd(64, 64, 4096, 4096)       # H*W*C beyond the kernel's offset range
    try:
        ops.set_conv_algorithm("winograd")
        assert ops._use_winograd(8, 4, 9, 9) and not ops._use_winograd(64, 64, 4096, 4096)
        ops.set_conv_algorithm("direct")
        assert not ops._use_winograd(64, 64, 224, 224)
        with pytest.raises(ValueError):
            ops.set_conv_algorithm("fft")
    finally:
        ops.set_conv_algorithm("auto")


def test_argument_validation_of_the_sequence_and_pooling_entry_points():
    """Bad arguments are rejected on the host, before any launch: these calls need no GPU."""
    lib = _cabi.lib()
    p = ctypes.c_void_p(4096)      # any non-null, 16-byte aligned address: never dereferenced
    odd = ctypes.c_void_p(4100)
    E = _cabi.PipedreamAmdError
    # label smoothing: empty shapes, NULL pointers, ld < V, non-positive divisor
    with pytest.raises(E, match="empty"):
        lib.pd_label_smoothing_fwd_f32(p, p, p, p, p, 0, 10, 10, 0, 0.1, 1.0, None)
    with pytest.raises(E, match="NULL"):
        lib.pd_label_smoothing_fwd_f32(p, None, p, p, p, 4, 10, 10, 0, 0.1, 1.0, None)
    with pytest.raises(E, match="ld < V"):
        lib.pd_label_smoothing_fwd_f32(p, p, p, p, p, 4, 10, 8, 0, 0.1, 1.0, None)
    with pytest.raises(E, match="divisor"):
        lib.pd_label_smoothing_bwd_f32(p, p, p, p, p, 4, 10, 10, 10, 0, 0.1, 0.0, None)
    with pytest.raises(E, match="leading dimension"):
        lib.pd_label_smoothing_bwd_f32(p, p, p, p, p, 4, 10, 10, 9, 0, 0.1, 1.0, None)
    # revert_varlen / length mask: nothing to do is fine; in-place reversal, odd sizes and pitches are not
    lib.pd_revert_varlen(None, None, None, 0, 5, 64, 64, 64, None)
    with pytest.raises(E, match="in place"):
        lib.pd_revert_varlen(p, p, p, 3, 2, 64, 64, 64, None)
    with pytest.raises(E, match="pitch"):
        lib.pd_revert_varlen(p, ctypes.c_void_p(8192), p, 3, 2, 64, 32, 64, None)
    with pytest.raises(E, match="2-byte"):
        lib.pd_length_mask_apply(p, p, p, 3, 2, 7, 7, 7, None)
    with pytest.raises(E, match="NULL"):
        lib.pd_length_mask_apply(p, p, None, 3, 2, 64, 64, 64, None)
    with pytest.raises(E, match="65535"):
        lib.pd_revert_varlen(p, ctypes.c_void_p(8192), p, 70000, 2, 64, 64, 64, None)
    # the host-side mask builder works on host memory
    lengths = (ctypes.c_int64 * 3)(3, 2, 1)
    mask = (ctypes.c_uint8 * 9)()
    lib.pd_set_mask_u8(ctypes.cast(lengths, ctypes.c_void_p), 3, 3, ctypes.cast(mask, ctypes.c_void_p))
    assert list(mask) == [1, 1, 1, 1, 1, 0, 1, 0, 0]
    with pytest.raises(E, match="NULL"):
        lib.pd_set_mask_u8(None, 3, 3, ctypes.cast(mask, ctypes.c_void_p))
    # pooling with index bytes: channel multiple of 4, alignment, NULL
    with pytest.raises(E, match="multiple of 4"):
        lib.pd_maxpool2x2_fwd_idx_nhwc_f32(p, p, p, 1, 4, 4, 6, 0, None)
    with pytest.raises(E, match="aligned"):
        lib.pd_maxpool2x2_fwd_idx_nhwc_f32(odd, p, p, 1, 4, 4, 8, 0, None)
    with pytest.raises(E, match="NULL"):
        lib.pd_maxpool2x2_bwd_idx_nhwc_f32(p, p, None, 1, 4, 4, 8, 0, None)
    lib.pd_maxpool2x2_fwd_idx_nhwc_f32(None, None, None, 1, 1, 3, 8, 0, None)      # no window: nothing to do
    # convolution with the pooling epilogue: shapes and pointers
    with pytest.raises(E, match="2x2 window"):
        lib.pd_conv3x3_winograd_fwd_pool_nhwc_f32(p, p, None, p, p, 1, 1, 8, 16, 32, 1, None)
    with pytest.raises(E, match="NULL"):
        lib.pd_conv3x3_winograd_fwd_pool_nhwc_f32(p, p, None, None, p, 1, 8, 8, 16, 32, 1, None)
    with pytest.raises(E, match="C % 8"):
        lib.pd_conv3x3_winograd_fwd_pool_nhwc_f32(p, p, None, p, p, 1, 8, 8, 12, 32, 1, None)
    with pytest.raises(E, match="too large"):
        lib.pd_conv3x3_winograd_fwd_nhwc_f32(p, p, None, None, None, p, 1, 4096, 4096, 64, 64, 0, None)
    # ... and with the pooling backward in its epilogue
    with pytest.raises(E, match="NULL"):
        lib.pd_conv3x3_winograd_fwd_unpool_nhwc_f32(p, p, None, p, p, 1, 8, 8, 16, 32, None)
    with pytest.raises(E, match="too large"):
        lib.pd_conv3x3_winograd_fwd_unpool_nhwc_f32(p, p, p, p, p, 1, 2048, 2048, 64, 64, None)
    # Winograd weight gradient: channel counts, a batch whose pixels overflow its 32-bit row counter, workspace
    with pytest.raises(E, match="unsupported channel counts"):
        lib.pd_conv3x3_winograd_wgrad_nhwc_f32(p, p, p, p, p, 1 << 30, 1, 8, 8, 48, 64, None)
    with pytest.raises(E, match="too many pixels"):
        lib.pd_conv3x3_winograd_wgrad_nhwc_f32(p, p, p, p, p, 1 << 30, 70000, 224, 224, 64, 64, None)
    with pytest.raises(E, match="workspace too small"):
        lib.pd_conv3x3_winograd_wgrad_nhwc_f32(p, p, p, p, p, 1024, 1, 8, 8, 64, 64, None)
