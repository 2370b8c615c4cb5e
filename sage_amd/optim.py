"""Optimizers: host-side mirror of optim.rs.

As in the reference an update is a handful of map expressions per parameter, evaluated eagerly
(optim.rs:128-131 "eager-execution like mode"); nothing here has a kernel of its own.  `grads` is the
{parameter: gradient Var} mapping of `grad_param`; every gradient must already hold its value (the
reference warns and evaluates it inside the optimizer otherwise, optim.rs:55-58, 144-147; so do we).

One deliberate difference: the new value is copied INTO the parameter's existing buffer instead of
replacing the parameter's tensor (optim.rs:92, 173), so a compiled `Program` that was recorded on
that buffer keeps seeing the current weights when it is replayed.

Reference behaviour that is kept because results would differ otherwise:
* `Adam` stores all-zero first and second moments on the first update of a gradient and starts
  accumulating on the second (optim.rs:149-163), and divides by 1 - beta^t with t starting at 1
  and growing once per update call (optim.rs:165-176).  The first update therefore leaves the
  parameters unchanged (0 / (0 + eps)).
* `Sgd` with momentum != 0 indexes a missing entry on first use (optim.rs:67-69: the `contains_key`
  test is inverted) and panics; here that is a KeyError.  Plain SGD (momentum 0) works.
"""
import ctypes as C

from .tensor import Tensor
from .var import Var, evaluate, params_changed, scalar


def _one_minus(x):
    """1 - x as the reference forms it: its hyper-parameters are f32 fields and `1.0 - self.beta1` is an f32
    subtraction (optim.rs:152, 160; 1 - 0.999f = 0.0009999871, not 0.001f)."""
    import numpy as np
    return float(np.float32(1.0) - np.float32(x))


def _value(grad, ctx):
    if grad.value is None:
        evaluate(ctx, [grad])
    return grad.value


def _assign(param, new_tensor, ctx):
    """param <- new value, in place (see the module docstring)."""
    old = param.value
    if old is None or not old.is_dense() or old.extents != new_tensor.extents or not new_tensor.is_dense():
        param.set(new_tensor)
        return
    params_changed()
    lib = ctx._lib
    ctx.check(lib.sg_memcpy_d2d(ctx.handle, C.c_void_p(old.buf.ptr + old.shape.offset * 4),
                                C.c_void_p(new_tensor.buf.ptr + new_tensor.shape.offset * 4), old.size() * 4))


def _compile(ctx, pairs):
    """pairs: [(expression Var, destination Tensor)].  One Program that evaluates every expression and then
    copies each result into its destination; building it performs the step once."""
    from .var import Program
    prog = Program(ctx, [e for e, _ in pairs])
    lib = ctx._lib
    for out, (_, dest) in zip(prog.outputs, pairs):
        args = (C.c_void_p(dest.buf.ptr + dest.shape.offset * 4), C.c_void_p(out.buf.ptr + out.shape.offset * 4), C.c_uint64(dest.size() * 4))
        ctx.check(lib.sg_memcpy_d2d(ctx.handle, *args))
        prog.calls.append((lib.sg_memcpy_d2d, args, [out, dest]))
    prog.changes_params = True
    params_changed()
    return prog


class Optimizer:
    def init(self, ctx):
        raise NotImplementedError

    def update(self, grads, ctx):
        raise NotImplementedError

    def compile(self, grads, ctx):
        """The update of `update(grads, ctx)` as a replayable `Program` (which can also be captured into a
        HIP graph): same expressions, evaluated once per `run()` on fixed buffers, with the state and the
        parameters rewritten in place.  Building it performs one update.  The reference has no
        counterpart: its optimizers rebuild and evaluate their expressions on every step."""
        raise NotImplementedError


class Sgd(Optimizer):
    """optim.rs:14-96."""

    def __init__(self, lr, momentum=0.0, dampening=0.0, weight_decay=0.0, nesterov=False):
        self.lr, self.momentum, self.dampening = float(lr), float(momentum), float(dampening)
        self.weight_decay, self.nesterov = float(weight_decay), bool(nesterov)
        self.b, self.g = {}, {}

    def init(self, ctx):
        self.b.clear()
        self.g.clear()

    def update(self, grads, ctx):
        for param, grad in grads.items():
            if not param.is_data():
                raise TypeError("param is not data tensor")
            gv = Var.new(_value(grad, ctx))
            g = gv + param * self.weight_decay if self.weight_decay != 0.0 else gv
            if self.momentum != 0.0:
                if id(grad) not in self.b:
                    b = Var.new(self.b[id(grad)]) * self.momentum + g * _one_minus(self.dampening)  # optim.rs:67-69
                else:
                    b = g
                self.b[id(grad)] = b.eval(ctx)
                b = Var.new(self.b[id(grad)])
                g = Var.new(self.g[id(grad)]) + b * self.momentum if self.nesterov and id(grad) in self.g else b
                self.g[id(grad)] = g.eval(ctx)
                g = Var.new(self.g[id(grad)])
            _assign(param, (param - g * self.lr).eval(ctx), ctx)

    def compile(self, grads, ctx):
        if self.momentum != 0.0:
            raise KeyError("Sgd with momentum fails in the reference (optim.rs:67-69)")
        pairs = []
        for param, grad in grads.items():
            gv = Var.new(_value(grad, ctx))
            g = gv + param * self.weight_decay if self.weight_decay != 0.0 else gv
            pairs.append((param - g * self.lr, param.value))
        return _compile(ctx, pairs)


class Adam(Optimizer):
    """optim.rs:98-178."""

    def __init__(self, lr, beta1=0.9, beta2=0.999, eps=1e-08, weight_decay=0.0):
        self.lr, self.beta1, self.beta2, self.eps = float(lr), float(beta1), float(beta2), float(eps)
        self.weight_decay = float(weight_decay)
        self.t = None
        self.m_t, self.v_t = {}, {}

    def init(self, ctx):
        import numpy as np
        self.m_t.clear()
        self.v_t.clear()
        self.t = Tensor.from_numpy(ctx, np.ones(1, np.float32))

    def update(self, grads, ctx):
        if self.t is None:
            self.init(ctx)
        t = Var.new(self.t)
        for param, grad in grads.items():
            if not param.is_data():
                raise TypeError("param is not data tensor")
            gv = Var.new(_value(grad, ctx))
            g = gv + param * self.weight_decay if self.weight_decay != 0.0 else gv
            key = id(grad)
            if key in self.m_t:
                m_t = Var.new(self.m_t[key]) * self.beta1 + g * _one_minus(self.beta1)
            else:
                m_t = scalar(0.0, grad.extents)
            self.m_t[key] = m_t.eval(ctx)
            m_t = Var.new(self.m_t[key])
            if key in self.v_t:
                v_t = Var.new(self.v_t[key]) * self.beta2 + g.pow(2.0) * _one_minus(self.beta2)
            else:
                v_t = scalar(0.0, grad.extents)
            self.v_t[key] = v_t.eval(ctx)
            v_t = Var.new(self.v_t[key])
            m_hat = m_t / (-scalar(self.beta1, [1]).pow(t) + 1.0)
            v_hat = v_t / (-scalar(self.beta2, [1]).pow(t) + 1.0)
            _assign(param, (param - m_hat * self.lr / (v_hat.sqrt() + self.eps)).eval(ctx), ctx)
        self.t = (t + 1.0).eval(ctx)

    def compile(self, grads, ctx, fused=True):
        """fused=True (default, when every tensor is dense fp32): all parameters are updated by sg_adam_update,
        one launch per 32 of them, followed by t <- t + 1.  fused=False replays the reference's operators: three
        map kernels and three copies per parameter.  Both give the same bits."""
        if self.t is None or any(id(g) not in self.m_t for g in grads.values()):
            raise RuntimeError("Adam.compile needs the state of every gradient: call update() once first "
                               "(the first update creates all-zero moments, optim.rs:149-163)")
        t = Var.new(self.t)
        if fused and self._fusable(grads, ctx):
            return self._compile_fused(grads, ctx, t)
        pairs = []
        for param, grad in grads.items():
            gv = Var.new(_value(grad, ctx))
            g = gv + param * self.weight_decay if self.weight_decay != 0.0 else gv
            key = id(grad)
            m_t = Var.new(self.m_t[key]) * self.beta1 + g * _one_minus(self.beta1)
            v_t = Var.new(self.v_t[key]) * self.beta2 + g.pow(2.0) * _one_minus(self.beta2)
            m_hat = m_t / (-scalar(self.beta1, [1]).pow(t) + 1.0)
            v_hat = v_t / (-scalar(self.beta2, [1]).pow(t) + 1.0)
            pairs += [(m_t, self.m_t[key]), (v_t, self.v_t[key]),
                      (param - m_hat * self.lr / (v_hat.sqrt() + self.eps), param.value)]
        pairs.append((t + 1.0, self.t))
        return _compile(ctx, pairs)

    def _fusable(self, grads, ctx):
        from . import abi
        for param, grad in grads.items():
            ts = (param.value, _value(grad, ctx), self.m_t[id(grad)], self.v_t[id(grad)])
            if any(x is None or x.dtype != abi.FLOAT or not x.is_dense() or x.extents != ts[0].extents for x in ts):
                return False
        return True

    def _compile_fused(self, grads, ctx, t):
        from . import abi
        lib = ctx._lib
        n = len(grads)
        cols = [[], [], [], []]
        for param, grad in grads.items():
            for col, x in zip(cols, (param.value, grad.value, self.m_t[id(grad)], self.v_t[id(grad)])):
                col.append(x)
        arrays = [(abi.sg_tensor * max(n, 1))(*[x.c() for x in col]) for col in cols]
        hyper = abi.sg_adam_hyper(self.lr, self.beta1, self.beta2, _one_minus(self.beta1), _one_minus(self.beta2), self.eps, self.weight_decay)
        step = self.t.c()
        prog = _compile(ctx, [])
        args = (C.c_int(n), *arrays, C.byref(step), C.byref(hyper))
        ctx.check(lib.sg_adam_update(ctx.handle, *args))
        prog.calls.append((lib.sg_adam_update, args, [cols, arrays, hyper, step, self.t]))
        # t <- t + 1 behind the update (which reads it)
        tail = _compile(ctx, [(t + 1.0, self.t)])
        prog.calls += tail.calls
        prog.keep = tail
        return prog
