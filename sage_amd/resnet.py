"""ResNet: host-side mirror of models/resnet.rs (basic-block variants; BatchNorm is commented out in
the reference, resnet.rs:80-83, so there is none here either).  Activations are NHWC."""
from . import nn
from .layers import AdaptiveAvgPool2d, Conv2d, Dense, Flatten, Layer, MaxPool2d, Relu, Sequential


class ResNetConfig:
    """resnet.rs:11-73."""

    def __init__(self, chan_input, num_classes, num_blocks, expansion, use_bottleneck):
        self.chan_input, self.num_classes = chan_input, num_classes
        self.num_blocks, self.expansion, self.use_bottleneck = num_blocks, expansion, use_bottleneck

    @staticmethod
    def d18(chan_input, num_classes):
        return ResNetConfig(chan_input, num_classes, [2, 2, 2, 2], 1, False)

    @staticmethod
    def d34(chan_input, num_classes):
        return ResNetConfig(chan_input, num_classes, [3, 4, 6, 3], 1, False)

    @staticmethod
    def d50(chan_input, num_classes):
        return ResNetConfig(chan_input, num_classes, [3, 4, 6, 3], 4, True)

    @staticmethod
    def d101(chan_input, num_classes):
        return ResNetConfig(chan_input, num_classes, [3, 4, 23, 3], 4, True)

    @staticmethod
    def d152(chan_input, num_classes):
        return ResNetConfig(chan_input, num_classes, [3, 8, 36, 3], 4, True)


class BasicLayer(Layer):
    """resnet.rs:155-176, 270-279."""

    def __init__(self, in_planes, planes, stride, config):
        out_planes = config.expansion * planes
        self.main = Sequential(Conv2d(in_planes, planes, 3, stride, 1, 1), Relu(), Conv2d(planes, out_planes, 3, 1, 1, 1))
        self.downsample = None
        if stride != 1 or in_planes != out_planes:
            self.downsample = Sequential(Conv2d(in_planes, out_planes, 1, stride, 0, 1))

    def params(self):
        return self.main.params() + (self.downsample.params() if self.downsample else [])

    def pass_(self, x):
        y_long = self.main.pass_(x)
        y = y_long + (self.downsample.pass_(x) if self.downsample else x)
        return nn.relu(y)


class BottleneckLayer(BasicLayer):
    """resnet.rs:178-243: 1x1 -> 3x3 (stride) -> 1x1 (expansion), same shortcut rule as the basic block."""

    def __init__(self, in_planes, planes, stride, config):
        out_planes = config.expansion * planes
        self.main = Sequential(Conv2d(in_planes, planes, 1), Relu(), Conv2d(planes, planes, 3, stride, 1, 1), Relu(),
                               Conv2d(planes, out_planes, 1))
        self.downsample = None
        if stride != 1 or in_planes != out_planes:
            self.downsample = Sequential(Conv2d(in_planes, out_planes, 1, stride, 0, 1))


class ResNet(Layer):
    """resnet.rs:75-130."""

    def __init__(self, config):
        block = BottleneckLayer if config.use_bottleneck else BasicLayer
        m = Sequential()
        in_planes = 64
        out_planes = in_planes
        m.add(Conv2d(config.chan_input, in_planes, 7, 2, 3, 1))
        m.add(Relu())
        m.add(MaxPool2d(3, 2, 1, 1))
        for i in range(4):
            stride = 1 if i == 0 else 2
            ip = in_planes
            for b in range(config.num_blocks[i]):
                m.add(block(ip, out_planes, stride if b == 0 else 1, config))
                ip = out_planes * config.expansion
            in_planes = out_planes * config.expansion
            out_planes *= 2
        m.add(AdaptiveAvgPool2d([1, 1]))
        m.add(Flatten())
        m.add(Dense(512 * config.expansion, config.num_classes))
        self.model = m

    def params(self):
        return self.model.params()

    def pass_(self, x):
        return self.model.pass_(x)
