"""Forward pass of a sage_amd layer tree evaluated with the CPU oracle's operators (test helper).

Walks the same layer objects the GPU path runs, but computes every layer with the oracle's un-fused
restatements, so a whole model can be checked end to end without a second hand-written copy of it."""
import numpy as np

from oracle import oracle as O
from sage_amd import densenet, layers, mobilenet, resnet


def host(v):
    return O.HT.from_numpy(v.value.numpy())


def forward(layer, x):
    if isinstance(layer, (resnet.ResNet, densenet.DenseNet, mobilenet.MobileNetV2)):
        return forward(layer.model, x)
    if isinstance(layer, layers.Sequential):
        for l in layer.layers:
            x = forward(l, x)
        return x
    if isinstance(layer, layers.Conv2d):
        return O.conv2d_layer(x, host(layer.weight), host(layer.bias), layer.stride, layer.padding, layer.dilation)
    if isinstance(layer, layers.Dense):
        return O.dense(x, host(layer.weight), host(layer.bias))
    if isinstance(layer, layers.Relu):
        return O.relu(x)
    if isinstance(layer, layers.AvgPool2d):  # before MaxPool2d: it is a subclass
        return O.avg_pool_2d(x, layer.k, layer.s, layer.p, layer.d)
    if isinstance(layer, layers.MaxPool2d):
        return O.max_pool_2d(x, layer.k, layer.s, layer.p, layer.d)
    if isinstance(layer, layers.AdaptiveAvgPool2d):
        return O.adaptive_avg_pool_2d(x, layer.extents)
    if isinstance(layer, layers.Flatten):
        return x.view([x.extents[0], -1])
    if isinstance(layer, resnet.BasicLayer):  # covers resnet.BottleneckLayer
        y = forward(layer.main, x)
        sc = forward(layer.downsample, x) if layer.downsample else x
        return O.relu(O.binary("add", y, sc))
    if isinstance(layer, densenet.BottleneckLayer):
        return O.concat([x, forward(layer.main, x)], 3)
    if isinstance(layer, mobilenet.InvertedResidual):
        y = forward(layer.main, x)
        return O.binary("add", x, y) if layer.shortcut else y
    raise TypeError(f"no oracle rule for {type(layer).__name__}")
