"""MobileNetV2: host-side mirror of models/mobilenet.rs.  The reference's inverted residual is built
from ORDINARY convolutions (no depthwise grouping) and its 3x3 stage is `Conv2d::with(hidden, hidden,
3, stride, 0, 0)`: padding 0 and DILATION 0 (mobilenet.rs:113), so all nine taps read the same pixel and
the spatial size only shrinks through the stride.  Kept as is."""
from .layers import AdaptiveAvgPool2d, Conv2d, Dense, Flatten, Layer, Relu, Sequential


def make_divisible(val, div, min_val):
    """mobilenet.rs:10-18."""
    new_val = max(min_val, (val + div // 2) // div * div)
    return new_val + div if float(new_val) < 0.9 * float(val) else new_val


class MobileNetV2Config:
    """mobilenet.rs:20-35."""

    def __init__(self, chan_in, num_classes, width_mul=1):
        self.chan_in, self.num_classes, self.width_mul = chan_in, num_classes, width_mul


class InvertedResidual(Layer):
    """mobilenet.rs:100-136."""

    def __init__(self, inp, oup, stride, expand_ratio):
        hidden = inp * expand_ratio
        m = Sequential()
        if expand_ratio != 1:
            m.add(Conv2d(inp, hidden, 1, 1, 0, 1))
            m.add(Relu())
        m.add(Conv2d(hidden, hidden, 3, stride, 0, 0))
        m.add(Relu())
        m.add(Conv2d(hidden, oup, 1, 1, 0, 1))
        self.main = m
        self.shortcut = stride == 1 and inp == oup

    def params(self):
        return self.main.params()

    def pass_(self, x):
        return x + self.main.pass_(x) if self.shortcut else self.main.pass_(x)


class MobileNetV2(Layer):
    """mobilenet.rs:37-84."""

    CFG = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]

    def __init__(self, config):
        chan_in = make_divisible(32 * config.width_mul, 8, 8)
        m = Sequential()
        m.add(Conv2d(config.chan_in, chan_in, 3, 2, 1, 1))
        m.add(Relu())
        for t, c, n, s in self.CFG:
            chan_out = make_divisible(c * config.width_mul, 8, 8)
            for i in range(n):
                m.add(InvertedResidual(chan_in, chan_out, s if i == 0 else 1, t))
                chan_in = chan_out
        chan_out = make_divisible(1280 * config.width_mul, 8, 8)
        m.add(Conv2d(chan_in, chan_out, 1))
        m.add(Relu())
        m.add(AdaptiveAvgPool2d([1, 1]))
        m.add(Flatten())
        m.add(Dense(chan_out, config.num_classes))
        self.model = m

    def params(self):
        return self.model.params()

    def pass_(self, x):
        return self.model.pass_(x)
