"""Stage module definitions in the format of the reference's generated model packages
(e.g. runtime/image_classification/models/vgg16/gpus=4_straight/__init__.py:13-20):
``model(criterion)`` returns ``[(stage_module, [input names], [output names]), ...,
(criterion, [..], ["loss"])]``."""
