"""DenseNet: host-side mirror of models/densenet.rs.  Activations are NHWC; as in the reference there
is no batch normalisation in the blocks (densenet.rs:131-135 builds relu -> 1x1 conv -> 3x3 conv) and
the dropout probability of the configuration is never used."""
from .layers import AdaptiveAvgPool2d, AvgPool2d, Conv2d, Dense, Flatten, Layer, Relu, Sequential
from .var import concat


class DenseNetConfig:
    """densenet.rs:10-54."""

    def __init__(self, chan_input, num_classes, depth, growth_rate, batch_norm_eps=0.0001, dropout_prob=0.2):
        self.chan_input, self.num_classes, self.depth, self.growth_rate = chan_input, num_classes, depth, growth_rate
        self.batch_norm_eps, self.dropout_prob = batch_norm_eps, dropout_prob

    @staticmethod
    def d121(chan_input, num_classes):
        return DenseNetConfig(chan_input, num_classes, 121, 12)

    @staticmethod
    def d169(chan_input, num_classes):
        return DenseNetConfig(chan_input, num_classes, 169, 24)

    @staticmethod
    def d201(chan_input, num_classes):
        return DenseNetConfig(chan_input, num_classes, 201, 12)


class BottleneckLayer(Layer):
    """densenet.rs:125-157: y = conv3x3(conv1x1(relu(x))); output = concat([x, y], channels)."""

    def __init__(self, in_planes, out_planes, config):
        inter = out_planes * 4
        self.main = Sequential(Relu(), Conv2d(in_planes, inter, 1, 1, 0, 1), Conv2d(inter, out_planes, 3, 1, 1, 1))

    def params(self):
        return self.main.params()

    def pass_(self, x):
        return concat([x, self.main.pass_(x)], 3)


class DenseNet(Layer):
    """densenet.rs:56-108."""

    def __init__(self, config):
        in_planes = 2 * config.growth_rate
        m = Sequential()
        m.add(Conv2d(config.chan_input, in_planes, 3, 1, 1, 1))
        n = (config.depth - 4) // 6
        for i in range(3):
            m.add(Sequential(*[BottleneckLayer(in_planes + j * config.growth_rate, config.growth_rate, config) for j in range(n)]))
            in_planes += n * config.growth_rate
            if i < 2:  # transition: relu -> 1x1 conv halving the channels -> 2x2 average pool
                m.add(Sequential(Relu(), Conv2d(in_planes, in_planes // 2, 1, 1, 0, 1), AvgPool2d(2)))
                in_planes //= 2
        m.add(Relu())
        m.add(AdaptiveAvgPool2d([1, 1]))
        m.add(Flatten())
        m.add(Dense(in_planes, config.num_classes))
        self.model = m

    def params(self):
        return self.model.params()

    def pass_(self, x):
        return self.model.pass_(x)
