"""Two-stage MLP 784 -> 1024 -> 1024 -> 10 (ReLU), split after the second layer: the
small CPU-runnable configuration.  The reference has no MLP model package; the layout
follows its generated packages (``StageN`` modules + ``model(criterion)``), the
initialisation is He-normal with zero biases."""
import torch

from .. import layers


def _he_init(module):
    for m in module.modules():
        if isinstance(m, layers.Linear):
            torch.nn.init.kaiming_normal_(m.weight, mode='fan_in', nonlinearity='relu')
            torch.nn.init.constant_(m.bias, 0)


class Stage0(torch.nn.Module):
    def __init__(self, d_in=784, d_hidden=1024):
        super(Stage0, self).__init__()
        self.layer1 = layers.Linear(d_in, d_hidden, relu=True)
        self.layer2 = layers.Linear(d_hidden, d_hidden, relu=True)
        _he_init(self)

    def forward(self, input0):
        return self.layer2(self.layer1(input0))


class Stage1(torch.nn.Module):
    def __init__(self, d_hidden=1024, d_out=10):
        super(Stage1, self).__init__()
        self.layer3 = layers.Linear(d_hidden, d_out)
        _he_init(self)

    def forward(self, input0):
        return self.layer3(input0)


def arch():
    return "mlp"


def model(criterion, d_in=784, d_hidden=1024, d_out=10):
    return [
        (Stage0(d_in, d_hidden), ["input0"], ["out0"]),
        (Stage1(d_hidden, d_out), ["out0"], ["out1"]),
        (criterion, ["out1"], ["loss"]),
    ]


def conf():
    """The mp_conf.json of this split (format of vgg16/gpus=4_straight/mp_conf.json)."""
    return {"module_to_stage_map": [0, 1, 1], "stage_to_rank_map": {"0": [0], "1": [1]}}
