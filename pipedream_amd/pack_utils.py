"""The two functions of the reference's compiled extension ``pack_utils._C``
(runtime/translation/seq2seq/csrc/pack_utils.cpp:35-38), under their names and argument conventions, on
the kernels of ``libpipedream_amd.so``::

    import pipedream_amd.pack_utils as C
    C.revert_varlen_tensor(input, lengths)     # seq2seq/models/encoder.py:17,21
    C.set_mask_cpp(lengths)                    # seq2seq/models/encoder.py:51
"""
import torch

from . import layers, ops


def revert_varlen_tensor(input, lengths):
    """``input`` [T, B, ...] on the GPU, ``lengths`` a 1-D CPU int64 tensor of B sequence lengths
    (pack_utils_kernel.cu:17-36).  Returns a new tensor in which every sequence is reversed in time over its
    own length, zeros behind it.  Every length must lie in (0, T]; the reference checks the last one only
    and reads out of bounds for a length above T."""
    if lengths.dim() != 1 or lengths.device.type != "cpu" or lengths.dtype != torch.int64:
        raise ValueError("'lengths' argument should be a 1D CPU int64 tensor")
    return ops.revert_varlen(input.contiguous(), layers._device_lengths(lengths, input, input.shape[0]))


def set_mask_cpp(lengths):
    """Host uint8 mask [lengths[0], B], 1 where ``lengths[b] > t`` (pack_utils.cpp:13-31)."""
    return ops.set_mask(lengths)
