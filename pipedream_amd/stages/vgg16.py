"""VGG16 stage definitions.

``model(criterion)`` / ``Stage0..Stage3`` follow the reference's 4-stage straight split
(runtime/image_classification/models/vgg16/gpus=4_straight/__init__.py:13-20,
stage0.py:10-33, stage1.py:8-32, stage2.py:8-36, stage3.py:10-46 and mp_conf.json): the
same layers in the same stages, the same attribute names for every layer that owns
parameters (so ``state_dict()`` keys match), the same initialisation.  A ReLU that
follows a convolution or a Linear layer inside a stage is fused into that layer's
epilogue, and the ReLU + MaxPool pair at the head of stages 1 is fused into the pooling
kernel, so those ReLU attributes do not exist as separate modules.

``FrontStage`` is the "conv1_1 .. pool2" stage of the headline benchmark configuration;
the reference never cuts exactly there (its 2-GPU split keeps conv1_1..conv2_2 in
vgg16/gpus=2/stage0.py:10-17 and puts the following ReLU + MaxPool at the head of
stage1.py:10-11), the layer names follow gpus=2/stage0.py.
"""
import torch

from .. import layers


def _initialize_weights(module):
    """stage0.py:22-33: conv kaiming-normal (fan_out, relu), biases 0, Linear N(0, 0.01)."""
    for m in module.modules():
        if isinstance(m, layers.Conv2d):
            w = torch.empty(m.weight.shape)
            torch.nn.init.kaiming_normal_(w, mode='fan_out', nonlinearity='relu')
            with torch.no_grad():
                m.weight.copy_(w)
                if m.bias is not None:
                    m.bias.zero_()
        elif isinstance(m, layers.Linear):
            torch.nn.init.normal_(m.weight, 0, 0.01)
            torch.nn.init.constant_(m.bias, 0)


class FrontStage(torch.nn.Module):
    """conv1_1, conv1_2, pool1, conv2_1, conv2_2, pool2 (ReLU after every convolution)."""

    def __init__(self):
        super(FrontStage, self).__init__()
        # a convolution with input_rectified=True masks its input gradient where its (rectified) input
        # is zero, so the convolution before it reads no mask either
        self.layer2 = layers.Conv2d(3, 64, relu=True, grad_premasked=True)
        # a pooling layer with relu=True is the identity on the rectified output of the convolution
        # before it and masks the gradient in its backward kernel, so that convolution's gradient
        # kernels read no mask (grad_premasked)
        # (with pool=True the convolution kernel pools in its epilogue; the pooling module keeps its place
        # in the layer list and passes the tensor through)
        # (a PoolGradLink between a pooling and the convolution behind it: the pooling's backward comes out
        # of that convolution's input-gradient kernel)
        pool1 = layers.PoolGradLink()
        self.layer4 = layers.Conv2d(64, 64, relu=True, input_rectified=True, pool=True, output_link=pool1)
        self.layer6 = layers.MaxPool2d(2, 2, relu=True, applied_by_producer=True)
        self.layer7 = layers.Conv2d(64, 128, relu=True, grad_premasked=True, input_link=pool1)
        self.layer9 = layers.Conv2d(128, 128, relu=True, input_rectified=True, pool=True)
        self.layer11 = layers.MaxPool2d(2, 2, relu=True, applied_by_producer=True)
        _initialize_weights(self)

    def forward(self, input0):
        out = self.layer4(self.layer2(input0))
        out = self.layer6(out)
        out = self.layer9(self.layer7(out))
        return self.layer11(out)


class Stage0(torch.nn.Module):
    def __init__(self):
        super(Stage0, self).__init__()
        self.layer2 = layers.Conv2d(3, 64, relu=True, grad_premasked=True)      # + layer3 ReLU; masked by layer4
        self.layer4 = layers.Conv2d(64, 64, input_rectified=True)
        _initialize_weights(self)

    def forward(self, input0):
        return self.layer4(self.layer2(input0))


class Stage1(torch.nn.Module):
    """Stage 1 of the 4-way split.  Its last ReLU's backward is applied by ``Stage2`` (the first convolution
    there masks its input gradient), so the gradient this stage receives must come from ``Stage2``:
    ``premasked_output_grads`` states it, ``StageRuntime`` checks it on every hand-off.
    ``plain_handoff=True`` builds the stage with the reference's contract instead: it takes dL/d(out) as
    runtime/communication.py:683-702 carries it and applies its last ReLU's backward itself."""

    def __init__(self, plain_handoff=False):
        super(Stage1, self).__init__()
        self.premasked_output_grads = (not plain_handoff,)
        pool1, pool2 = layers.PoolGradLink(), layers.PoolGradLink()
        self.layer2 = layers.MaxPool2d(2, 2, relu=True, link=pool1)    # layer1 ReLU + layer2 MaxPool
        self.layer3 = layers.Conv2d(64, 128, relu=True, grad_premasked=True, input_link=pool1)    # + layer4; masked by layer5
        self.layer5 = layers.Conv2d(128, 128, relu=True, input_rectified=True, pool=True,
                                    output_link=pool2)                  # + layer6 + layer7
        self.layer7 = layers.MaxPool2d(2, 2, relu=True, applied_by_producer=True)
        # layer8's ReLU is undone for the gradient by the next stage's first convolution (input_rectified)
        self.layer8 = layers.Conv2d(128, 256, relu=True, grad_premasked=not plain_handoff, input_link=pool2)   # + layer9
        _initialize_weights(self)

    def forward(self, input0):
        out = self.layer2(input0)
        out = self.layer5(self.layer3(out))
        return self.layer8(self.layer7(out))


class Stage2(torch.nn.Module):
    """Stage 2 of the 4-way split.  Takes ``Stage1``'s rectified output and applies that ReLU's backward to
    the gradient it hands back (``masks_input_grads``); its own last ReLU's backward is applied by the
    pooling layer that opens ``Stage3`` (``premasked_output_grads``).  ``plain_handoff=True``: neither; the
    stage hands back the gradient of its input as it is and masks the gradient it receives itself."""

    def __init__(self, plain_handoff=False):
        super(Stage2, self).__init__()
        self.masks_input_grads = (not plain_handoff,)
        self.premasked_output_grads = (not plain_handoff,)
        self.layer1 = layers.Conv2d(256, 256, relu=True, grad_premasked=True,
                                    input_rectified=not plain_handoff)   # + layer2; masked by layer3
        pool3 = layers.PoolGradLink()
        self.layer3 = layers.Conv2d(256, 256, relu=True, input_rectified=True, pool=True,
                                    output_link=pool3)                  # + layer4 + layer5
        self.layer5 = layers.MaxPool2d(2, 2, relu=True, applied_by_producer=True)
        self.layer6 = layers.Conv2d(256, 512, relu=True, grad_premasked=True, input_link=pool3)   # + layer7; masked by layer8
        self.layer8 = layers.Conv2d(512, 512, relu=True, grad_premasked=True, input_rectified=True)   # + layer9
        # layer10's ReLU is undone for the gradient by the next stage's pooling layer (relu=True)
        self.layer10 = layers.Conv2d(512, 512, relu=True, grad_premasked=not plain_handoff,
                                     input_rectified=True)  # + layer11
        _initialize_weights(self)

    def forward(self, input0):
        out = self.layer3(self.layer1(input0))
        out = self.layer5(out)
        return self.layer10(self.layer8(self.layer6(out)))


class Stage3(torch.nn.Module):
    """Last stage of the 4-way split; its opening ReLU + MaxPool applies the backward of ``Stage2``'s last
    ReLU (``masks_input_grads``).  ``plain_handoff=True``: a plain pooling layer (stage3.py:12), the
    gradient handed back is that of the stage's input."""

    def __init__(self, dropout=0.5, num_classes=1000, plain_handoff=False):
        super(Stage3, self).__init__()
        self.masks_input_grads = (not plain_handoff,)
        pool4 = layers.PoolGradLink()
        self.layer1 = layers.MaxPool2d(2, 2, relu=not plain_handoff, link=pool4)
        self.layer2 = layers.Conv2d(512, 512, relu=True, grad_premasked=True, input_link=pool4)   # + layer3; masked by layer4
        self.layer4 = layers.Conv2d(512, 512, relu=True, grad_premasked=True, input_rectified=True)   # + layer5
        self.layer6 = layers.Conv2d(512, 512, relu=True, input_rectified=True, pool=True)   # + layer7 + layer8
        self.layer8 = layers.MaxPool2d(2, 2, relu=True, applied_by_producer=True)
        self.flatten = layers.Flatten()
        self.layer11 = layers.Linear(25088, 4096, relu=True)   # + layer12
        self.layer13 = layers.Dropout(p=dropout)
        self.layer14 = layers.Linear(4096, 4096, relu=True)    # + layer15
        self.layer16 = layers.Dropout(p=dropout)
        self.layer17 = layers.Linear(4096, num_classes)
        _initialize_weights(self)

    def forward(self, input0):
        out = self.layer1(input0)
        out = self.layer6(self.layer4(self.layer2(out)))
        out = self.flatten(self.layer8(out))
        out = self.layer13(self.layer11(out))
        out = self.layer16(self.layer14(out))
        return self.layer17(out)


def arch():
    return "vgg16"


def model(criterion, dropout=0.5, plain_handoff=False):
    """The four stages and the criterion.  By default stages 1 -> 2 and 2 -> 3 exchange gradients that the
    consumer has already masked with the producer's last ReLU (one pass over the hand-off tensor saved per
    boundary; both sides declare it and ``StageRuntime`` checks it).  ``plain_handoff=True`` builds the same
    layers with the reference's contract on every boundary -- the gradient of the tensor that was sent,
    nothing applied to it -- for pipelines that mix these stages with stages from elsewhere."""
    return [
        (Stage0(), ["input0"], ["out0"]),
        (Stage1(plain_handoff=plain_handoff), ["out0"], ["out1"]),
        (Stage2(plain_handoff=plain_handoff), ["out1"], ["out2"]),
        (Stage3(dropout=dropout, plain_handoff=plain_handoff), ["out2"], ["out3"]),
        (criterion, ["out3"], ["loss"]),
    ]


def conf():
    """vgg16/gpus=4_straight/mp_conf.json"""
    return {"module_to_stage_map": [0, 1, 2, 3, 3],
            "stage_to_rank_map": {"0": [0], "1": [1], "2": [2], "3": [3]}}
