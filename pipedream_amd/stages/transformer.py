"""Transformer stage of the 2BW-style configuration: 6 pre-LN layers (hidden 1024, 16 heads,
FFN 4096, GELU), bf16 compute with fp32 master weights.

The reference's checked-out branch has no transformer model package (PipeDream-2BW lives on
another branch, README.md:7-8); the module follows the format of its generated stages
(``StageN`` module, ``model(criterion)`` list).  Input ``[batch, seq, hidden]`` in fp32 or
bf16, output bf16."""
import torch

from .. import layers


class Stage0(torch.nn.Module):
    def __init__(self, n_layers=6, hidden=1024, heads=16, ffn=4096):
        super(Stage0, self).__init__()
        self.layers = torch.nn.ModuleList([layers.TransformerLayer(hidden, heads, ffn) for _ in range(n_layers)])

    def forward(self, input0):
        x = layers.to_bf16(input0)
        for layer in self.layers:
            x = layer(x)
        return x


def arch():
    return "transformer"
