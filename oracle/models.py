"""CPU ORACLE -- test infrastructure, not product code.

``torch.nn`` twins of the stage definitions in ``pipedream_amd/stages``: same layer
order, same parameter names and the same random-number consumption at construction, so
that with one seed both sides start from identical weights.  Layer lists follow the
reference's generated stages where those exist (VGG16:
runtime/image_classification/models/vgg16/gpus=4_straight/stage0.py:10-33 ...
stage3.py:10-46; GNMT: runtime/translation/models/gnmt_large/gpus=4/stage0.py:10-40)."""
import torch


def _he_init(module):
    for m in module.modules():
        if isinstance(m, torch.nn.Linear):
            torch.nn.init.kaiming_normal_(m.weight, mode='fan_in', nonlinearity='relu')
            torch.nn.init.constant_(m.bias, 0)


class MlpStage0(torch.nn.Module):
    def __init__(self, d_in=784, d_hidden=1024):
        super(MlpStage0, self).__init__()
        self.layer1 = torch.nn.Linear(d_in, d_hidden)
        self.layer2 = torch.nn.Linear(d_hidden, d_hidden)
        _he_init(self)

    def forward(self, input0):
        return torch.relu(self.layer2(torch.relu(self.layer1(input0))))


class MlpStage1(torch.nn.Module):
    def __init__(self, d_hidden=1024, d_out=10):
        super(MlpStage1, self).__init__()
        self.layer3 = torch.nn.Linear(d_hidden, d_out)
        _he_init(self)

    def forward(self, input0):
        return self.layer3(input0)


# --------------------------------------------------------------------------------------
# VGG16 (layer lists of vgg16/gpus=4_straight/stage0-3.py and vgg16/gpus=2/stage0.py)
# --------------------------------------------------------------------------------------
def _vgg_init(module):
    """stage0.py:22-33"""
    for m in module.modules():
        if isinstance(m, torch.nn.Conv2d):
            torch.nn.init.kaiming_normal_(m.weight, mode='fan_out', nonlinearity='relu')
            if m.bias is not None:
                torch.nn.init.constant_(m.bias, 0)
        elif isinstance(m, torch.nn.Linear):
            torch.nn.init.normal_(m.weight, 0, 0.01)
            torch.nn.init.constant_(m.bias, 0)


def _conv(cin, cout):
    return torch.nn.Conv2d(cin, cout, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1))


class VggFrontStage(torch.nn.Module):
    """conv1_1 .. pool2"""

    def __init__(self):
        super(VggFrontStage, self).__init__()
        self.layer2 = _conv(3, 64)
        self.layer4 = _conv(64, 64)
        self.layer7 = _conv(64, 128)
        self.layer9 = _conv(128, 128)
        _vgg_init(self)

    def forward(self, x):
        F = torch.nn.functional
        x = F.relu(self.layer4(F.relu(self.layer2(x))))
        x = F.max_pool2d(x, 2, 2)
        x = F.relu(self.layer9(F.relu(self.layer7(x))))
        return F.max_pool2d(x, 2, 2)


class VggStage0(torch.nn.Module):
    def __init__(self):
        super(VggStage0, self).__init__()
        self.layer2 = _conv(3, 64)
        self.layer4 = _conv(64, 64)
        _vgg_init(self)

    def forward(self, x):
        return self.layer4(torch.relu(self.layer2(x)))


class VggStage1(torch.nn.Module):
    def __init__(self):
        super(VggStage1, self).__init__()
        self.layer3 = _conv(64, 128)
        self.layer5 = _conv(128, 128)
        self.layer8 = _conv(128, 256)
        _vgg_init(self)

    def forward(self, x):
        F = torch.nn.functional
        x = F.max_pool2d(F.relu(x), 2, 2)
        x = F.relu(self.layer5(F.relu(self.layer3(x))))
        return F.relu(self.layer8(F.max_pool2d(x, 2, 2)))


class VggStage2(torch.nn.Module):
    def __init__(self):
        super(VggStage2, self).__init__()
        self.layer1 = _conv(256, 256)
        self.layer3 = _conv(256, 256)
        self.layer6 = _conv(256, 512)
        self.layer8 = _conv(512, 512)
        self.layer10 = _conv(512, 512)
        _vgg_init(self)

    def forward(self, x):
        F = torch.nn.functional
        x = F.relu(self.layer3(F.relu(self.layer1(x))))
        x = F.max_pool2d(x, 2, 2)
        return F.relu(self.layer10(F.relu(self.layer8(F.relu(self.layer6(x))))))


class VggStage3(torch.nn.Module):
    """``masks``: optional callable (name, tensor) -> 0/1 keep-mask, so that a parity run can
    feed both sides the same dropout masks; without it dropout is torch's own."""

    def __init__(self, dropout=0.5, num_classes=1000, masks=None):
        super(VggStage3, self).__init__()
        self.layer2 = _conv(512, 512)
        self.layer4 = _conv(512, 512)
        self.layer6 = _conv(512, 512)
        self.layer11 = torch.nn.Linear(25088, 4096)
        self.layer14 = torch.nn.Linear(4096, 4096)
        self.layer17 = torch.nn.Linear(4096, num_classes)
        self.p = dropout
        self.masks = masks
        _vgg_init(self)

    def _drop(self, name, x):
        if not self.training or self.p == 0:
            return x
        if self.masks is None:
            return torch.nn.functional.dropout(x, self.p, True)
        return x * self.masks(name, x).to(x.dtype) * (1.0 / (1.0 - self.p))

    def forward(self, x):
        F = torch.nn.functional
        x = F.max_pool2d(x, 2, 2)
        x = F.relu(self.layer6(F.relu(self.layer4(F.relu(self.layer2(x))))))
        x = F.max_pool2d(x, 2, 2)
        x = x.reshape(x.size(0), -1)
        x = self._drop("layer13", F.relu(self.layer11(x)))
        x = self._drop("layer16", F.relu(self.layer14(x)))
        return self.layer17(x)


# --------------------------------------------------------------------------------------
# GNMT-style stage (gnmt_large/gpus=4/stage0.py:10-40 without the bidirectional layer)
# --------------------------------------------------------------------------------------
class GnmtStage0(torch.nn.Module):
    def __init__(self, vocab=32320, hidden=1024, dropout=0.2):
        super(GnmtStage0, self).__init__()
        self.layer6 = torch.nn.Embedding(vocab, hidden, padding_idx=0)
        self.layer7 = torch.nn.LSTM(hidden, hidden)
        self.layer8 = torch.nn.Dropout(p=dropout)
        self.layer9 = torch.nn.LSTM(hidden, hidden)
        self.layer11 = torch.nn.Dropout(p=dropout)
        self.layer12 = torch.nn.LSTM(hidden, hidden)
        self.layer15 = torch.nn.Dropout(p=dropout)
        self.layer16 = torch.nn.LSTM(hidden, hidden)

    def forward(self, input0):
        out6 = self.layer6(input0)
        out7 = self.layer7(out6)[0]
        out9 = self.layer9(self.layer8(out7))[0]
        out12 = self.layer12(self.layer11(out9))[0]
        out13 = out12 + out9
        out16 = self.layer16(self.layer15(out13))[0]
        return out16 + out13


class GnmtBidirStage0(torch.nn.Module):
    """gnmt_large/gpus=4/stage0.py:8-40 as generated (bidirectional first layer, two outputs)."""

    def __init__(self, vocab=32320, hidden=1024, dropout=0.2):
        super(GnmtBidirStage0, self).__init__()
        from . import seq2seq_oracle
        self.layer6 = torch.nn.Embedding(vocab, hidden, padding_idx=0)
        self.layer7 = seq2seq_oracle.EmuBidirLSTM(hidden, hidden)
        self.layer8 = torch.nn.Dropout(p=dropout)
        self.layer9 = torch.nn.LSTM(2 * hidden, hidden)
        self.layer11 = torch.nn.Dropout(p=dropout)
        self.layer12 = torch.nn.LSTM(hidden, hidden)
        self.layer15 = torch.nn.Dropout(p=dropout)
        self.layer16 = torch.nn.LSTM(hidden, hidden)
        self.layer19 = torch.nn.Dropout(p=dropout)
        self.layer20 = torch.nn.LSTM(hidden, hidden)

    def forward(self, input0, input1):
        out0 = input0.clone()
        out1 = input1.clone()
        out6 = self.layer6(out0)
        out7 = self.layer7(out6, out1)
        out10 = self.layer9(self.layer8(out7))[0]
        out13 = self.layer12(self.layer11(out10))[0] + out10
        out17 = self.layer16(self.layer15(out13))[0] + out13
        out21 = self.layer20(self.layer19(out17))[0]
        return (out17, out21)


# --------------------------------------------------------------------------------------
# bf16 pre-LN transformer stage (fp32 master parameters, bf16 activations and products)
# --------------------------------------------------------------------------------------
class TransformerLayerOracle(torch.nn.Module):
    """Same parameter names as pipedream_amd.layers.TransformerLayer.  Every product takes
    bf16 operands (weights rounded from the fp32 masters at use time); LayerNorm, softmax
    and GELU are evaluated by torch's bf16 CPU kernels (fp32 internally, bf16 results)."""

    def __init__(self, hidden, heads, ffn, eps=1e-5):
        super(TransformerLayerOracle, self).__init__()
        self.heads = heads
        self.ln1 = torch.nn.LayerNorm(hidden, eps=eps)
        self.qkv = torch.nn.Linear(hidden, 3 * hidden)
        self.proj = torch.nn.Linear(hidden, hidden)
        self.ln2 = torch.nn.LayerNorm(hidden, eps=eps)
        self.fc1 = torch.nn.Linear(hidden, ffn)
        self.fc2 = torch.nn.Linear(ffn, hidden)

    @staticmethod
    def _lin(x, m):
        return torch.nn.functional.linear(x, m.weight.bfloat16(), m.bias.bfloat16())

    @staticmethod
    def _ln(x, m):
        return torch.nn.functional.layer_norm(x.float(), x.shape[-1:], m.weight, m.bias, m.eps).bfloat16()

    def forward(self, x):
        B, S, H = x.shape
        d = H // self.heads
        qkv = self._lin(self._ln(x, self.ln1), self.qkv)
        q, k, v = [t.reshape(B, S, self.heads, d).transpose(1, 2) for t in qkv.split(H, dim=-1)]
        p = torch.softmax((q @ k.transpose(-1, -2)) * (1.0 / d ** 0.5), dim=-1)
        att = (p @ v).transpose(1, 2).reshape(B, S, H)
        x = self._lin(att, self.proj) + x
        f = torch.nn.functional.gelu(self._lin(self._ln(x, self.ln2), self.fc1))
        return self._lin(f, self.fc2) + x


class TransformerStage0(torch.nn.Module):
    def __init__(self, n_layers=6, hidden=1024, heads=16, ffn=4096):
        super(TransformerStage0, self).__init__()
        self.layers = torch.nn.ModuleList([TransformerLayerOracle(hidden, heads, ffn) for _ in range(n_layers)])

    def forward(self, x):
        x = x.bfloat16()
        for layer in self.layers:
            x = layer(x)
        return x
