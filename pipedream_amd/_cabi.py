"""ctypes binding of libpipedream_amd.so (the C ABI declared in include/pipedream_amd.h).

There is no CPU fallback: if the shared library has not been built the import of
any product module fails with a clear error, and every compute entry point needs a
HIP device.  Only the host-side integer bookkeeping (the version ring) runs without one.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpipedream_amd.so")

PD_OK = 0
# element formats of the mixed-precision optimizer step (include/pipedream_amd.h)
PD_F32, PD_BF16, PD_F16 = 0, 1, 2


class PipedreamAmdError(RuntimeError):
    """A C-ABI call returned non-zero."""

    def __init__(self, fn, code, msg):
        super().__init__("%s failed (code %d): %s" % (fn, code, msg))
        self.code = code


class TensorDesc(ctypes.Structure):
    """struct pd_tensor_desc"""
    _fields_ = [
        ("grad", ctypes.c_void_p),
        ("p_in", ctypes.c_void_p),
        ("p_out", ctypes.c_void_p),
        ("state0", ctypes.c_void_p),
        ("state1", ctypes.c_void_p),
        ("bf16_out", ctypes.c_void_p),
        ("n", ctypes.c_uint64),
    ]


_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_u64 = ctypes.c_uint64
_d = ctypes.c_double
_f = ctypes.c_float
_pi = ctypes.POINTER(ctypes.c_int)
_pi64 = ctypes.POINTER(ctypes.c_int64)
_pvp = ctypes.POINTER(ctypes.c_void_p)

# name -> (restype, argtypes, returns_status)
# Every symbol declared in include/pipedream_amd.h appears here; the CPU test-suite
# checks that the header and this table agree and that the library exports them all.
SIGNATURES = {
    "pd_abi_version": (_i, [], False),
    "pd_last_error": (ctypes.c_char_p, [], False),
    "pd_ring_create": (_i, [_vp, _u64, _i, _pvp], True),
    "pd_ring_destroy": (_i, [_vp], True),
    "pd_ring_num_versions": (_i, [_vp], False),
    "pd_ring_entry": (_i, [_vp, _i, _pi, _pi64], True),
    "pd_ring_slot_ptr": (_i, [_vp, _i, _pvp], True),
    "pd_ring_write_slot": (_i, [_vp, _pi], True),
    "pd_ring_push": (_i, [_vp, _i64, _pi], True),
    "pd_ring_broadcast": (_i, [_vp, _i, _u64, _vp], True),
    "pd_copy": (_i, [_vp, _vp, _u64, _vp], True),
    "pd_fill_zero": (_i, [_vp, _u64, _vp], True),
    "pd_sgd_step": (_i, [ctypes.POINTER(TensorDesc), _i, _d, _d, _d, _d, _i, _i, _d, _d, _vp], True),
    "pd_adam_step": (_i, [ctypes.POINTER(TensorDesc), _i, _d, _d, _d, _d, _d, _i64, _i, _d, _d, _vp], True),
    "pd_sgd_step_mixed": (_i, [ctypes.POINTER(TensorDesc), _i, _d, _d, _d, _d, _i, _i, _d, _d, _i, _i, _vp], True),
    "pd_adam_step_mixed": (_i, [ctypes.POINTER(TensorDesc), _i, _d, _d, _d, _d, _d, _i64, _i, _d, _d, _i, _i, _vp],
                           True),
    "pd_gemm_f32": (_i, [_i, _i, _i, _i, _i, _vp, _i, _vp, _i, _f, _vp, _i, _vp, _i, _vp], True),
    "pd_gemm_splitk_f32": (_i, [_i, _i, _i, _i, _i, _vp, _i, _vp, _i, _vp, _i, _vp], True),
    "pd_splitk_reduce_f32": (_i, [_vp, _i, _i, _i, _vp, _i, _f, _vp, _i, _vp], True),
    "pd_colsum_f32": (_i, [_vp, _vp, _u64, _i, _u64, _i, _f, _vp], True),
    "pd_relu_fwd_f32": (_i, [_vp, _vp, _u64, _vp], True),
    "pd_relu_bwd_f32": (_i, [_vp, _vp, _vp, _u64, _vp], True),
    "pd_mask_scale_f32": (_i, [_vp, _vp, _vp, _u64, _f, _vp], True),
    "pd_maxpool2x2_fwd_nhwc_f32": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp], True),
    "pd_maxpool2x2_bwd_nhwc_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp], True),
    "pd_xent_fwd_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i64, _vp], True),
    "pd_conv3x3_fwd_nhwc_f32": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp], True),
    "pd_conv3x3_filter_rot180_f32": (_i, [_vp, _vp, _i, _i, _vp], True),
    "pd_conv3x3_wgrad_workspace_bytes": (_i, [_i, _i, _i, _i, _i, ctypes.POINTER(ctypes.c_uint64)], True),
    "pd_conv3x3_dgrad_nhwc_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp], True),
    "pd_conv3x3_winograd_supported": (_i, [_i, _i], False),
    "pd_conv3x3_winograd_filter_bytes": (_i, [_i, _i, ctypes.POINTER(_u64)], True),
    "pd_conv3x3_winograd_filter_f32": (_i, [_vp, _vp, _i, _i, _i, _vp], True),
    "pd_conv3x3_winograd_set_pieces": (_i, [_i], True),
    "pd_conv3x3_winograd_set_wgrad_strips": (_i, [_i], True),
    "pd_conv3x3_winograd_fwd_nhwc_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp], True),
    "pd_conv3x3_winograd_fwd_pool_nhwc_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp], True),
    "pd_conv3x3_winograd_fwd_unpool_nhwc_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp], True),
    "pd_maxpool2x2_fwd_idx_nhwc_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp], True),
    "pd_maxpool2x2_bwd_idx_nhwc_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _vp], True),
    "pd_conv3x3_winograd_wgrad_supported": (_i, [_i, _i], False),
    "pd_conv3x3_winograd_wgrad_workspace_bytes": (_i, [_i, _i, ctypes.POINTER(_u64)], True),
    "pd_conv3x3_winograd_wgrad_nhwc_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _u64, _i, _i, _i, _i, _i, _vp], True),
    "pd_conv3x3_wgrad_nhwc_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _u64, _i, _i, _i, _i, _i, _vp], True),
    "pd_conv3x3_wgrad_noalloc_nhwc_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp], True),
    "pd_lstm_cell_fwd_f32": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp], True),
    "pd_lstm_cell_bwd_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _vp], True),
    "pd_lstm_recurrence_fwd_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _vp], True),
    "pd_lstm_recurrence_bwd_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _vp], True),
    "pd_add_f32": (_i, [_vp, _vp, _vp, _u64, _vp], True),
    "pd_embedding_fwd_f32": (_i, [_vp, _vp, _vp, _i, _i, _i64, _vp], True),
    "pd_embedding_bwd_f32": (_i, [_vp, _vp, _vp, _i, _i, _i64, _i64, _vp], True),
    "pd_gemm_bf16": (_i, [_i, _i, _i, _i, _i, _vp, _i, _vp, _i, _vp, _i, _i, _f, _f, _vp, _vp, _i, _i, _i,
                          ctypes.POINTER(ctypes.c_int64), _vp], True),
    "pd_gemm_bf16_set_tile": (_i, [_i, _i], True),
    "pd_split3_bf16_f32": (_i, [_vp, _i64, _i64, _i64, _vp, _i, _i, _vp], True),
    "pd_gemm_bf16_gelu": (_i, [_i, _i, _i, _i, _i, _i, _vp, _i, _vp, _i, _vp, _i, _vp, _vp, _i, _vp], True),
    "pd_layernorm_fwd_bf16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _vp], True),
    "pd_layernorm_bwd_partials": (_i, [_i], False),
    "pd_layernorm_bwd_bf16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _vp], True),
    "pd_attention_fwd_supported": (_i, [_i, _i], False),
    "pd_attention_fwd_bf16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp], True),
    "pd_attention_bwd_bf16": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp], True),
    "pd_softmax_fwd_bf16": (_i, [_vp, _vp, _i64, _i, _vp], True),
    "pd_softmax_bwd_bf16": (_i, [_vp, _vp, _vp, _i64, _i, _vp], True),
    "pd_gelu_fwd_bf16": (_i, [_vp, _vp, _u64, _vp], True),
    "pd_gelu_bwd_bf16": (_i, [_vp, _vp, _vp, _u64, _vp], True),
    "pd_add_bf16": (_i, [_vp, _vp, _vp, _u64, _vp], True),
    "pd_cast_f32_to_bf16": (_i, [_vp, _vp, _u64, _vp], True),
    "pd_cast_bf16_to_f32": (_i, [_vp, _vp, _u64, _vp], True),
    "pd_colsum_bf16": (_i, [_vp, _vp, _u64, _i, _u64, _i, _vp], True),
    "pd_colsum_batch_workspace_floats": (_i, [_i, _vp, _vp, _i, ctypes.POINTER(_u64)], True),
    "pd_colsum_batch": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _u64, _i, _vp], True),
    "pd_label_smoothing_fwd_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i64, _i64, _f, _f, _vp], True),
    "pd_label_smoothing_bwd_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i64, _i64, _i64, _f, _f, _vp], True),
    "pd_revert_varlen": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp], True),
    "pd_length_mask_apply": (_i, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp], True),
    "pd_set_mask_u8": (_i, [_vp, _i64, _i64, _vp], True),
    "pd_xent_bwd_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i64, _vp], True),
}


class _Lib:
    def __init__(self, path):
        if not os.path.isfile(path):
            raise ImportError(
                "pipedream_amd: %s is missing. Build it with "
                "`make -C pipedream_amd/csrc` (needs hipcc); there is no CPU fallback." % path)
        self._dll = ctypes.CDLL(path)
        self._raw = {}
        for name, (restype, argtypes, _) in SIGNATURES.items():
            fn = getattr(self._dll, name)  # AttributeError here = symbol not exported
            fn.restype = restype
            fn.argtypes = argtypes
            self._raw[name] = fn
        got = self._raw["pd_abi_version"]()
        if got != 1:
            raise ImportError("pipedream_amd: ABI version %d, expected 1" % got)

    def last_error(self):
        msg = self._raw["pd_last_error"]()
        return msg.decode("utf-8", "replace") if msg else ""

    def raw(self, name):
        return self._raw[name]

    def __getattr__(self, name):
        try:
            fn = self._raw[name]
        except KeyError:
            raise AttributeError(name)
        checked = SIGNATURES[name][2]
        if not checked:
            return fn

        def call(*args):
            rc = fn(*args)
            if rc != PD_OK:
                raise PipedreamAmdError(name, rc, self.last_error())
            return rc

        call.__name__ = name
        self.__dict__[name] = call
        return call


_lib = None


def lib():
    """The loaded library (loads on first use)."""
    global _lib
    if _lib is None:
        _lib = _Lib(LIB_PATH)
    return _lib


def stream_ptr(stream=None):
    """hipStream_t of a torch stream (default: the current one) as a void*."""
    import torch
    if stream is None:
        stream = torch.cuda.current_stream()
    return ctypes.c_void_p(stream.cuda_stream)


def require_device(t, what="tensor"):
    """Compute entry points only take HIP device tensors."""
    if not t.is_cuda:
        raise RuntimeError(
            "pipedream_amd: %s lives on %s; the HIP kernels need a GPU tensor and "
            "there is no CPU fallback" % (what, t.device))
    return t
