"""Layers: host-side mirror of layers.rs (the types BERT and ResNet-18 are made of).

Each layer owns its parameters as data `Var`s and composes operators in `pass_`, exactly as the
reference's `Layer::pass` does.  The reference's quirks are kept and cited: LayerNorm ignores its
eps argument and uses 1e-05 with scalar gamma = beta = 1 (layers.rs:563-590), Dropout is the
identity (layers.rs:605-609), weights are [in, out] (layers.rs:215).
"""
import numpy as np

from . import nn
from .tensor import FLOAT, Tensor
from .var import Var, _pair, avg_pool_2d, conv_2d, into_var, max_pool_2d


def _set(ctx, var, array):
    var.set(Tensor.from_numpy(ctx, np.asarray(array, np.float32).reshape(var.extents)))


def kaiming_uniform(rng, extents, gain=1.0):
    """tensor/init.rs:6-15."""
    std = gain * np.sqrt(1.0 / fan_in_out(extents)[0])
    a = np.sqrt(3.0) * std
    return rng.uniform(-a, a, extents).astype(np.float32)


def kaiming_normal(rng, extents, gain=1.0):
    """tensor/init.rs:17-25."""
    std = gain * np.sqrt(1.0 / fan_in_out(extents)[0])
    return (rng.standard_normal(extents) * std).astype(np.float32)


class Layer:
    def params(self):
        return []

    def init(self, ctx, rng):
        """Parameter::init: fill this layer's parameters.  `rng` is a numpy Generator; the reference draws
        from the host's thread_rng, so its values are not reproducible and only the distributions are mirrored."""
        for v in vars(self).values():
            for l in (v if isinstance(v, (list, tuple)) else [v]):
                if isinstance(l, Layer):
                    l.init(ctx, rng)

    def pass_(self, x):
        raise NotImplementedError

    def __call__(self, x):
        return self.pass_(x)


def fan_in_out(extents):
    """tensor/init.rs:27-50: dim0 = receptive field * ... as the reference computes it: for
    [d0, d1, rest...] fan_in = d1 * prod(rest), fan_out = d0 * prod(rest)."""
    rest = 1
    for e in extents[2:]:
        rest *= e
    return extents[1] * rest, extents[0] * rest


class Dense(Layer):
    """layers.rs:208-247."""

    def __init__(self, dim_in, dim_out):
        self.weight = Var.empty([dim_in, dim_out]).name("dense.weight")
        self.bias = Var.empty([dim_out]).name("dense.bias")

    def params(self):
        return [self.weight, self.bias]

    def init(self, ctx, rng):
        """layers.rs:224-236."""
        _set(ctx, self.weight, kaiming_uniform(rng, self.weight.extents))
        _set(ctx, self.bias, np.zeros(self.bias.extents))

    def pass_(self, x):
        return (into_var(x).matmul(self.weight) + self.bias).name("dense")


class Conv2d(Layer):
    """layers.rs:327-404: weight [KH,KW,C,OC]; kernel_size/stride/padding/dilation pairs are [w,h]."""

    def __init__(self, chan_in, chan_out, kernel_size, stride=1, padding=0, dilation=1):
        k = _pair(kernel_size)
        self.weight = Var.empty([k[1], k[0], chan_in, chan_out]).name("conv2d.weight")
        self.bias = Var.empty([chan_out]).name("conv2d.bias")
        self.stride, self.padding, self.dilation = _pair(stride), _pair(padding), _pair(dilation)

    def params(self):
        return [self.weight, self.bias]

    def init(self, ctx, rng):
        """layers.rs:374-386."""
        _set(ctx, self.weight, kaiming_normal(rng, self.weight.extents))
        _set(ctx, self.bias, np.zeros(self.bias.extents))

    def pass_(self, x):
        return (conv_2d(x, self.weight, self.stride, self.padding, self.dilation) + self.bias).name("conv_2d")


class Embedding(Layer):
    """layers.rs:406-463: ids -> view [B*L,1] -> expand [B*L,E] (stride 0) -> gather(weight, ., 0)."""

    def __init__(self, num_embeddings, embedding_dim):
        self.num_embeddings, self.embedding_dim = num_embeddings, embedding_dim
        self.weight = Var.empty([num_embeddings, embedding_dim]).name("embedding.weight")

    def params(self):
        return [self.weight]

    def init(self, ctx, rng):
        """layers.rs:466-472: standard normal."""
        _set(ctx, self.weight, rng.standard_normal(self.weight.extents))

    def pass_(self, idx):
        idx = into_var(idx)
        e = self.embedding_dim
        if idx.rank > 1:
            b, l = idx.extent(0), idx.extent(1)
            i = idx.view([b * l, 1]).expand([b * l, e])
            return self.weight.gather(i, 0).view([b, l, e]).name("embedding")
        l = idx.extent(0)
        i = idx.view([l, 1]).expand([l, e])
        return self.weight.gather(i, 0).view([l, e]).name("embedding")


class LayerNorm(Layer):
    """layers.rs:548-590.  reference_exact=True (default): gamma, beta are [1] tensors and eps is
    the hard-coded 1e-05 whatever was asked for (layers.rs:588).  reference_exact=False: per-feature
    gamma/beta of `features` elements and the eps given — the configuration BERT checkpoints use."""

    def __init__(self, axes, eps, features=None, reference_exact=True):
        self.axes = [axes] if isinstance(axes, int) else list(axes)
        self.eps = 1e-05 if reference_exact else float(eps)
        n = 1 if reference_exact or features is None else features
        self.gamma = Var.empty([n]).name("layer_norm.gamma")
        self.beta = Var.empty([n]).name("layer_norm.beta")

    def params(self):
        return [self.gamma, self.beta]

    def init(self, ctx, rng):
        """layers.rs:570-578: gamma = beta = 1 (also beta)."""
        _set(ctx, self.gamma, np.ones(self.gamma.extents))
        _set(ctx, self.beta, np.ones(self.beta.extents))

    def pass_(self, x):
        return nn.layer_norm(x, self.axes, self.gamma, self.beta, self.eps).name("layer_norm")


class Softmax(Layer):
    """layers.rs:249-273."""

    def __init__(self, axes):
        self.axes = [axes] if isinstance(axes, int) else list(axes)

    def pass_(self, x):
        return nn.softmax(x, self.axes).name("softmax")


class Relu(Layer):
    def pass_(self, x):
        return nn.relu(x)


class Gelu(Layer):
    def pass_(self, x):
        return nn.gelu(x)


class Dropout(Layer):
    """layers.rs:593-609: not implemented in the reference; identity."""

    def __init__(self, prob):
        self.prob = prob

    def pass_(self, x):
        return into_var(x)


class Flatten(Layer):
    """layers.rs:196-206."""

    def pass_(self, x):
        x = into_var(x)
        return x.view([x.extent(0), -1]).name("flatten")


class MaxPool2d(Layer):
    """layers.rs:295-326."""

    def __init__(self, kernel_size, stride=None, padding=0, dilation=1):
        self.k = _pair(kernel_size)
        self.s = _pair(stride) if stride is not None else list(self.k)
        self.p, self.d = _pair(padding), _pair(dilation)

    def pass_(self, x):
        return max_pool_2d(x, self.k, self.s, self.p, self.d).name("max_pool_2d")


class AvgPool2d(MaxPool2d):
    def pass_(self, x):
        return avg_pool_2d(x, self.k, self.s, self.p, self.d).name("avg_pool_2d")


class AdaptiveAvgPool2d(Layer):
    """layers.rs:124-154: stride = in/out, kernel = in - (out-1)*stride."""

    def __init__(self, extents):
        self.extents = _pair(extents)

    def pass_(self, x):
        x = into_var(x)
        iw, ih = x.extent(2), x.extent(1)
        ow, oh = self.extents
        stride = [iw // ow, ih // oh]
        ker = [iw - (ow - 1) * stride[0], ih - (oh - 1) * stride[1]]
        return avg_pool_2d(x, ker, stride, [0, 0], [1, 1]).name("adaptive_avg_pool_2d")


class BatchNorm2d(Layer):
    """layers.rs:479-548: scalar gamma and beta, per-channel running statistics, all initialised to one; the
    pass normalises with the RUNNING statistics (there is no batch-statistics path in the reference)."""

    def __init__(self, num_features, eps):
        self.num_features, self.eps = num_features, float(eps)
        self.gamma = Var.empty([1]).name("batch_norm_2d.gamma")
        self.beta = Var.empty([1]).name("batch_norm_2d.beta")
        self.running_mean = Var.empty([num_features]).name("batch_norm_2d.running_mean")
        self.running_var = Var.empty([num_features]).name("batch_norm_2d.running_var")

    def params(self):
        return [self.gamma, self.beta]

    def init(self, ctx, rng):
        _set(ctx, self.gamma, np.ones(1))
        _set(ctx, self.beta, np.ones(1))
        _set(ctx, self.running_mean, np.ones(self.num_features))
        _set(ctx, self.running_var, np.ones(self.num_features))

    def pass_(self, x):
        from .var import batch_norm_2d
        # the eps given to the constructor is ignored: the pass hard-codes 1e-05 (layers.rs:541-543)
        return batch_norm_2d(x, self.gamma, self.beta, self.running_mean, self.running_var, 1e-05).name("batch_norm_2d")


class Sequential(Layer):
    """layers.rs:275-326."""

    def __init__(self, *layers):
        self.layers = list(layers)

    def add(self, layer):
        self.layers.append(layer)
        return self

    def params(self):
        return [p for l in self.layers for p in l.params()]

    def pass_(self, x):
        for l in self.layers:
            x = l.pass_(x)
        return x


def load_params(ctx, layer, arrays):
    """Set every parameter of `layer` (in params() order) from host arrays."""
    ps = layer.params()
    if len(ps) != len(arrays):
        raise ValueError(f"{len(ps)} parameters, {len(arrays)} arrays")
    for p, a in zip(ps, arrays):
        a = np.asarray(a, dtype=np.float32)
        if list(a.shape) != p.extents:
            raise ValueError(f"{p.label}: expected {p.extents}, got {list(a.shape)}")
        p.set(Tensor.from_numpy(ctx, a))
