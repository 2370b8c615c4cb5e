"""sage_amd — MI355X (gfx950) backend for Sage's operator hot path, with a host-side mirror of the
reference's front-end (Shape, Tensor, Var, nn, layers, BERT, ResNet) on top of the C ABI in
include/sage_hip.h.  All compute runs in sage_amd/libsage_hip.so; there is no CPU fallback."""
from . import abi, bert, densenet, grad, layers, mobilenet, nn, optim, resnet, var  # noqa: F401
from .shape import Shape  # noqa: F401
from .tensor import FLOAT, INT, UINT, Context, Tensor  # noqa: F401
from .var import Program, Var, evaluate, set_fusion  # noqa: F401
