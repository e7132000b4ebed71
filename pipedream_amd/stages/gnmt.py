"""GNMT-style encoder stage: embedding + 4 uni-directional LSTM layers with residual
connections around the last two, dropout in front of every LSTM.

Layer list and residual pattern follow the reference's
runtime/translation/models/gnmt_large/gpus=4/stage0.py:10-40 with the bidirectional first
layer (``EmuBidirLSTM``, stage0.py:11) replaced by a plain ``LSTM(1024, 1024)``, which is
what the GNMT configuration of the benchmark names (4 uni-directional layers).  Attribute
names of parameter-owning layers are the reference's (layer6 embedding, layer9/12/16/20
LSTMs) plus layer7 for the substituted first LSTM."""
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


def arch():
    return "gnmt"
