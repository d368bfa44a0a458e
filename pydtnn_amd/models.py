"""Model definitions for the networks the benchmark and the tests run, in the form of the reference's
``pydtnn/models/*.py``: a function that adds the layers to a ``Model``.

``create_vgg16_imagenet`` follows pydtnn/models/vgg16.py (its two Dropout(0.5) layers are optional: the
benchmark's configuration has none); ``create_resnet50_imagenet`` follows
pydtnn/models/resnet50_imagenet.py:25-69 (v1.5: a downsampling block strides its 3x3 convolution).
"""
from .layers import (AdditionBlock, AveragePool2D, BatchNormalization, Conv2D, Dropout, FC, Flatten, Input,
                     MaxPool2D, Relu)


def create_vgg16_imagenet(model, dropout=False, initializer="he_normal"):
    model.add(Input(shape=(224, 224, 3)))
    for convs, filters in ((2, 64), (2, 128), (3, 256), (3, 512), (3, 512)):
        for _ in range(convs):
            model.add(Conv2D(nfilters=filters, filter_shape=(3, 3), padding=1, stride=1, activation="relu",
                             weights_initializer=initializer))
        model.add(MaxPool2D(pool_shape=(2, 2), stride=2))
    model.add(Flatten())
    for width in (4096, 4096):
        model.add(FC(shape=(width,), activation="relu", weights_initializer=initializer))
        if dropout:
            model.add(Dropout(rate=0.5))
    model.add(FC(shape=(1000,), activation="softmax", weights_initializer=initializer))
    return model


def bottleneck(filters, stride, projection, initializer="he_uniform"):
    """One ResNet bottleneck: 1x1 -> 3x3 (strided when downsampling) -> 1x1 to 4*filters, each followed by
    BatchNormalization, summed with the input (through a strided 1x1 projection where the shape changes)."""
    def conv(n, k, s=1, p=0):
        return Conv2D(nfilters=n, filter_shape=(k, k), stride=s, padding=p, weights_initializer=initializer)

    main = [conv(filters, 1), BatchNormalization(), Relu(),
            conv(filters, 3, stride, 1), BatchNormalization(), Relu(),
            conv(4 * filters, 1), BatchNormalization()]
    shortcut = [conv(4 * filters, 1, stride), BatchNormalization()] if projection else []
    return AdditionBlock(main, shortcut)


def create_resnet50_imagenet(model, stages=((64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)), classes=1000,
                             input_shape=(224, 224, 3)):
    model.add(Input(shape=input_shape))
    model.add(Conv2D(nfilters=64, filter_shape=(7, 7), stride=2, padding=3, weights_initializer="he_uniform"))
    model.add(MaxPool2D(pool_shape=(3, 3), stride=2, padding=1))
    for filters, blocks, first_stride in stages:
        for i in range(blocks):
            model.add(bottleneck(filters, first_stride if i == 0 else 1, projection=i == 0))
            model.add(Relu())
    model.add(AveragePool2D(pool_shape=(0, 0)))
    model.add(Flatten())
    model.add(FC(shape=(classes,), activation="softmax"))
    return model
