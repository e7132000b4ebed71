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
