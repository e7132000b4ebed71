"""CPU ORACLE -- test infrastructure, not product code.

Restatement of the translation-stage pieces the HIP kernels of ``pd_seq2seq.hip`` replace:

* ``label_smoothing``      -- LabelSmoothing.forward, runtime/translation/seq2seq/train/smoothing.py:23-34
* ``revert_varlen_offsets``/``revert_varlen`` -- revert_varlen_tensor and its kernel,
  runtime/translation/seq2seq/csrc/pack_utils_kernel.cu:7-62
* ``set_mask``             -- set_mask_cpp, runtime/translation/seq2seq/csrc/pack_utils.cpp:13-31
* ``EmuBidirLSTM``         -- runtime/translation/seq2seq/models/encoder.py:13-64 (the two-layer form)

Pinned (tests/test_oracle_seq2seq.py) by: ``torch.nn.functional.cross_entropy`` with and without
``label_smoothing`` (sum reduction, ``ignore_index``), a float64 evaluation of -sum_j q_j log p_j with the
smoothed target distribution, the closed form log V for constant logits; per-sequence ``flip`` for
revert_varlen and its involution property; an ``arange`` comparison for the mask; and
``torch.nn.LSTM(bidirectional=True)`` on packed sequences for the bidirectional layer.  The reference holds
no golden vectors for any of these."""
import numpy as np
import torch


def label_smoothing(output, target, padding_idx, smoothing):
    """The criterion of smoothing.py:23-34: fp32 log-softmax over the last dimension of the [T, B, V] logits
    (:24-25); per row the negative log-probability of the target (:28) and the negative mean log-probability
    (:30), mixed with weights 1 - smoothing and smoothing (:31); rows whose target is the padding index are
    dropped (:27, :29-30); the sum over the other rows is divided by the batch size B (:32-33)."""
    rows = output.reshape(-1, output.shape[-1])
    logp = torch.log_softmax(rows, dim=-1, dtype=torch.float32)
    keep = target.ne(padding_idx)
    picked = logp[torch.arange(rows.shape[0]), target]
    per_row = (1.0 - smoothing) * (-picked) + smoothing * (-logp.mean(dim=-1))
    return per_row[keep].sum() / output.shape[1]


def revert_varlen_offsets(lengths, seq_length, batch_size, feature_size):
    """The host-side table of pack_utils_kernel.cu:37-52: for every (t, i) the element offset of the source
    row, or -1 for positions behind the end of sequence i."""
    offsets = []
    for t in range(seq_length):
        for i in range(batch_size):
            if lengths[i] > t:
                offsets.append(i * feature_size + (lengths[i] - t - 1) * batch_size * feature_size)
            else:
                offsets.append(-1)
    return offsets


def revert_varlen(x, lengths):
    """pack_utils_kernel.cu:7-13 applied with the table above: out row r = in[offset_r : offset_r + F], or the
    pad value 0 (:56) where the offset is negative."""
    lengths = [int(v) for v in lengths]
    seq_length, batch_size = x.shape[0], x.shape[1]
    if len(lengths) != batch_size:
        raise ValueError("Expected `len(lengths)` to be equal to batch_size")
    if batch_size and lengths[batch_size - 1] <= 0:                                       # :33-35
        raise ValueError("Length of all samples has to be greater than 0")
    flat = x.detach().contiguous().cpu().numpy().reshape(-1)
    feature_size = flat.size // max(seq_length * batch_size, 1)
    out = np.zeros_like(flat)
    for row, off in enumerate(revert_varlen_offsets(lengths, seq_length, batch_size, feature_size)):
        if off >= 0:
            out[row * feature_size:(row + 1) * feature_size] = flat[off:off + feature_size]
    return torch.from_numpy(out.reshape(tuple(x.shape)))


def set_mask(lengths):
    """pack_utils.cpp:13-31: uint8 [lengths[0], B], 1 where lengths[i] > t."""
    lengths = [int(v) for v in lengths]
    batch_size = len(lengths)
    seq_length = lengths[0] if batch_size else 0
    out = torch.empty((seq_length, batch_size), dtype=torch.uint8)
    for t in range(seq_length):
        for i in range(batch_size):
            out[t, i] = 1 if lengths[i] > t else 0
    return out


class _RevertVarlen(torch.autograd.Function):
    """encoder.py:13-21"""

    @staticmethod
    def forward(ctx, input, lengths):
        ctx.lengths = lengths
        return revert_varlen(input, lengths)

    @staticmethod
    def backward(ctx, grad_output):
        return revert_varlen(grad_output, ctx.lengths), None


class EmuBidirLSTM(torch.nn.Module):
    """encoder.py:25-64, the ``emu_bidir_lstm`` form at every batch size (the reference's other branch, for
    batches above 128, is torch's packed bidirectional LSTM -- the routine this class is pinned against)."""

    def __init__(self, input_size, hidden_size):
        super(EmuBidirLSTM, self).__init__()
        self.bidir = torch.nn.LSTM(input_size, hidden_size, 1, True, False, bidirectional=True)     # :31
        self.layer1 = torch.nn.LSTM(input_size, hidden_size, 1, True, False)                        # :32
        self.layer2 = torch.nn.LSTM(input_size, hidden_size, 1, True, False)                        # :33
        for name in ("weight_ih_l0", "weight_hh_l0", "bias_ih_l0", "bias_hh_l0"):                   # :34-41
            setattr(self.layer1, name, getattr(self.bidir, name))
            setattr(self.layer2, name, getattr(self.bidir, name + "_reverse"))

    def forward(self, input, lengths):
        """encoder.py:50-57 and :59: the backward direction runs on the sequences reversed over their own
        lengths and its output is reversed back; the forward direction's output is zeroed behind every
        sequence's end; both halves side by side."""
        lengths = lengths.cpu().long()
        keep = set_mask(lengths)
        # the reference builds the mask with lengths[0] rows and multiplies a [T, B, H] tensor with it (:51,
        # :55), so the longest sequence must fill the tensor
        assert keep.shape[0] == input.shape[0], "the longest sequence must fill the tensor"
        backward_dir = self.layer2(_RevertVarlen.apply(input, lengths))[0]
        forward_dir = self.layer1(input)[0] * keep.unsqueeze(-1).type_as(input)
        return torch.cat([forward_dir, _RevertVarlen.apply(backward_dir, lengths)], dim=2)
