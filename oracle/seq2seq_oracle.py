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
    """smoothing.py:23-34, line by line."""
    confidence = 1.0 - smoothing
    x = output.view(output.size(0) * output.size(1), -1)                                  # :24
    logprobs = torch.nn.functional.log_softmax(x, dim=-1, dtype=torch.float32)            # :25
    non_pad_mask = (target != padding_idx)                                                # :27
    nll_loss = -logprobs.gather(dim=-1, index=target.unsqueeze(1))                        # :28
    nll_loss = nll_loss.squeeze(1)[non_pad_mask]                                          # :29
    smooth_loss = -logprobs.mean(dim=-1)[non_pad_mask]                                    # :30
    loss = confidence * nll_loss + smoothing * smooth_loss                                # :31
    loss = loss.sum()                                                                     # :32
    loss = loss / output.size(1)                                                          # :33
    return loss


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
        lengths = lengths.cpu().long()                                                              # :59
        mask = set_mask(lengths)
        # :51 builds the mask with lengths[0] rows; it multiplies a [T, B, H] tensor, so T == lengths[0]
        assert mask.shape[0] == input.shape[0], "the longest sequence must fill the tensor"
        mask = mask.unsqueeze(-1).type_as(input)
        inputl1 = _RevertVarlen.apply(input, lengths)                                               # :52
        out1 = self.layer2(inputl1)                                                                 # :53
        outputs = _RevertVarlen.apply(out1[0], lengths)                                             # :54
        out0 = self.layer1(input)[0] * mask                                                         # :55
        return torch.cat([out0, outputs], dim=2)                                                    # :56
