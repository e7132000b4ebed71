"""GNMT-style encoder stage: embedding + 4 uni-directional LSTM layers with residual
connections around the last two, dropout in front of every LSTM.

Layer list and residual pattern follow the reference's
runtime/translation/models/gnmt_large/gpus=4/stage0.py:10-40 with the bidirectional first
layer (``EmuBidirLSTM``, stage0.py:11) replaced by a plain ``LSTM(1024, 1024)``, which is
what the GNMT configuration of the benchmark names (4 uni-directional layers).  Attribute
names of parameter-owning layers are the reference's (layer6 embedding, layer9/12/16/20
LSTMs) plus layer7 for the substituted first LSTM.

``BidirStage0`` is the reference's stage as generated, bidirectional first layer included:
two inputs (token ids, sequence lengths), two outputs (stage0.py:21-40)."""
import torch

from .. import layers


class Stage0(torch.nn.Module):
    def __init__(self, vocab=32320, hidden=1024, dropout=0.2):
        super(Stage0, self).__init__()
        self.layer6 = layers.Embedding(vocab, hidden, padding_idx=0)
        self.layer7 = layers.LSTM(hidden, hidden)
        self.layer8 = layers.Dropout(p=dropout)
        self.layer9 = layers.LSTM(hidden, hidden)
        self.layer11 = layers.Dropout(p=dropout)
        self.layer12 = layers.LSTM(hidden, hidden)
        self.layer15 = layers.Dropout(p=dropout)
        self.layer16 = layers.LSTM(hidden, hidden)

    def forward(self, input0):
        out6 = self.layer6(input0)                      # [T, B, H]
        out7 = self.layer7(out6)[0]
        out9 = self.layer9(self.layer8(out7))[0]
        out12 = self.layer12(self.layer11(out9))[0]
        out13 = layers.add(out12, out9)
        out16 = self.layer16(self.layer15(out13))[0]
        return layers.add(out16, out13)


class BidirStage0(torch.nn.Module):
    """runtime/translation/models/gnmt_large/gpus=4/stage0.py:8-40: embedding, ``EmuBidirLSTM``, three
    LSTM layers (residual connection around the second and third) and the first LSTM of the next group;
    returns ``(out17, out21)`` like the reference.  The reference's ``input.clone()`` copies at the head of
    the stage (stage0.py:22-23) are not made: nothing here writes its inputs."""

    def __init__(self, vocab=32320, hidden=1024, dropout=0.2):
        super(BidirStage0, self).__init__()
        self.layer6 = layers.Embedding(vocab, hidden, padding_idx=0)
        self.layer7 = layers.EmuBidirLSTM(hidden, hidden)
        self.layer8 = layers.Dropout(p=dropout)
        self.layer9 = layers.LSTM(2 * hidden, hidden)
        self.layer11 = layers.Dropout(p=dropout)
        self.layer12 = layers.LSTM(hidden, hidden)
        self.layer15 = layers.Dropout(p=dropout)
        self.layer16 = layers.LSTM(hidden, hidden)
        self.layer19 = layers.Dropout(p=dropout)
        self.layer20 = layers.LSTM(hidden, hidden)

    def forward(self, input0, input1):
        out6 = self.layer6(input0)                      # [T, B, H]
        out7 = self.layer7(out6, input1)                # [T, B, 2H]
        out10 = self.layer9(self.layer8(out7))[0]
        out12 = self.layer12(self.layer11(out10))[0]
        out13 = layers.add(out12, out10)
        out16 = self.layer16(self.layer15(out13))[0]
        out17 = layers.add(out16, out13)
        out21 = self.layer20(self.layer19(out17))[0]
        return (out17, out21)


def arch():
    return "gnmt"
