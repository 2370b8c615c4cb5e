"""Context and device tensors: host-side mirror of session/context.rs, session/device.rs, tensor.rs.

A `Context` owns the backend context (device, stream, kernel cache, allocator); a `Tensor` is a
descriptor (`Shape` + dtype) over a reference-counted device buffer, so layout operators are
zero-copy exactly as in the reference (core.rs:249-260, 315-317, 395-397).
"""
import ctypes as C

import numpy as np

from . import abi
from .shape import Shape, default_strides

FLOAT, INT, UINT = abi.FLOAT, abi.INT, abi.UINT
_NP_OF = {FLOAT: np.float32, INT: np.int32, UINT: np.uint32}
_DT_OF = {np.dtype(np.float32): FLOAT, np.dtype(np.int32): INT, np.dtype(np.uint32): UINT}


# Bumped whenever existing device data may have been rewritten in place from the host side or by an
# optimizer; caches of data derived from parameters (var.py) compare against it.
_PARAM_EPOCH = [0]


class Context:
    """Context::with_device (context.rs:43-52).  capacity=None: bounded by the device only;
    capacity=abi.REFERENCE_CAPACITY_BYTES reproduces the reference's 1000 MiB allocator cap.
    use_cache / use_sub_buffer are the two switches of Allocator::new (memory.rs:64-69): the reference's Context
    passes (False, True), every request then being a device allocation of its own; use_cache=True serves requests
    from chunks (Pool's caching branch) and the capacity then bounds the bytes of the chunks held."""

    def __init__(self, device=0, capacity=None, use_cache=False, use_sub_buffer=True):
        self._lib = abi.lib()
        h = C.c_void_p()
        rc = self._lib.sg_ctx_create_pooled(int(device), int(capacity or 0), int(bool(use_cache)), int(bool(use_sub_buffer)), C.byref(h))
        if rc != abi.OK:
            raise abi.SageError(rc, f"sg_ctx_create(device={device}) failed: no usable HIP device")
        self.handle = h
        self.launches = 0  # operator launches issued through this context

    def close(self):
        if self.handle:
            self._lib.sg_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def check(self, rc):
        abi.check(self.handle, rc)

    def sync(self):
        self.check(self._lib.sg_sync(self.handle))

    def stream(self):
        return self._lib.sg_stream(self.handle)

    def mem_stats(self):
        v = [C.c_uint64() for _ in range(4)]
        self.check(self._lib.sg_mem_stats(self.handle, *[C.byref(x) for x in v]))
        return dict(zip(("used", "reserved", "peak", "capacity"), (x.value for x in v)))

    def kernel_cache_size(self):
        return self._lib.sg_kernel_cache_size(self.handle)

    def trim(self):
        self.check(self._lib.sg_trim(self.handle))


class Buffer:
    """One device allocation, freed when the last tensor viewing it goes away (memory.rs:685-692)."""

    def __init__(self, ctx, nbytes):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        ctx.check(ctx._lib.sg_alloc(ctx.handle, self.nbytes, C.byref(p)))
        self.ptr = p.value

    def __del__(self):
        ctx = getattr(self, "ctx", None)
        if ctx is not None and ctx.handle and getattr(self, "ptr", None):
            ctx._lib.sg_free(ctx.handle, C.c_void_p(self.ptr))
            self.ptr = None


class Tensor:
    """TensorDesc + shared device data (tensor.rs:38-41, 107-110)."""

    def __init__(self, buf, dtype, shape):
        self.buf = buf
        self.dtype = dtype
        self.shape = shape

    # ---- construction / readback (Tensor::new + to_device, tensor.rs:280-309; Buffer::read)
    @staticmethod
    def from_numpy(ctx, a):
        a = np.asarray(a)
        if a.dtype == np.float64:
            a = a.astype(np.float32)
        elif a.dtype == np.int64:
            a = a.astype(np.int32)
        if a.dtype not in _DT_OF:
            raise abi.DTypeError(abi.ERR_DTYPE, f"unsupported host dtype {a.dtype}")
        a = np.ascontiguousarray(a)
        ext = list(a.shape) if a.ndim else [1]
        t = Tensor.uninit(ctx, ext, _DT_OF[a.dtype])
        ctx.check(ctx._lib.sg_memcpy_h2d(ctx.handle, C.c_void_p(t.buf.ptr), a.ctypes.data_as(C.c_void_p), a.nbytes))
        return t

    @staticmethod
    def uninit(ctx, extents, dtype=FLOAT):
        """Tensor::uninit (tensor.rs:195-206): numel * 4 bytes (device.rs:75)."""
        sh = Shape(extents)
        return Tensor(Buffer(ctx, max(1, sh.size()) * 4), dtype, sh)

    def copy_from_numpy(self, a):
        """Overwrite this (dense) tensor's elements with `a` (Buffer::write, device.rs:111-128)."""
        ctx = self.buf.ctx
        a = np.ascontiguousarray(np.asarray(a, dtype=_NP_OF[self.dtype]))
        if list(a.shape) != self.shape.extents or not self.is_dense():
            raise abi.ShapeError(abi.ERR_SHAPE, "copy_from_numpy needs a dense tensor of the same extents")
        dst = C.c_void_p(self.buf.ptr + self.shape.offset * 4)
        ctx.check(ctx._lib.sg_memcpy_h2d(ctx.handle, dst, a.ctypes.data_as(C.c_void_p), a.nbytes))
        _PARAM_EPOCH[0] += 1

    def numpy(self):
        """Blocking read of the whole buffer, then the strided view is taken on the host."""
        ctx = self.buf.ctx
        n = self.buf.nbytes // 4
        host = np.empty(n, dtype=_NP_OF[self.dtype])
        ctx.check(ctx._lib.sg_memcpy_d2h(ctx.handle, host.ctypes.data_as(C.c_void_p), C.c_void_p(self.buf.ptr), n * 4))
        v = np.lib.stride_tricks.as_strided(host[self.shape.offset:], shape=self.shape.extents,
                                            strides=[s * 4 for s in self.shape.strides])
        return np.array(v)

    @property
    def ctx(self):
        return self.buf.ctx

    @property
    def extents(self):
        return self.shape.extents

    @property
    def strides(self):
        return self.shape.strides

    @property
    def offset(self):
        return self.shape.offset

    @property
    def rank(self):
        return self.shape.rank

    def size(self):
        return self.shape.size()

    def with_shape(self, shape):
        return Tensor(self.buf, self.dtype, shape)

    def c(self):
        """The sg_tensor descriptor handed across the C ABI."""
        t = abi.sg_tensor()
        t.base = self.buf.ptr
        t.dtype = self.dtype
        t.rank = self.shape.rank
        for i in range(self.shape.rank):
            t.extents[i] = self.shape.extents[i]
            t.strides[i] = self.shape.strides[i]
        t.offset = self.shape.offset
        return t

    def is_dense(self):
        return self.shape.strides == default_strides(self.shape.extents)

    @staticmethod
    def all_close(a, b, eps):
        """Tensor::all_close (tensor.rs:320-328): max |a-b| < eps."""
        a = a.numpy() if isinstance(a, Tensor) else np.asarray(a)
        b = b.numpy() if isinstance(b, Tensor) else np.asarray(b)
        return a.shape == b.shape and float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64)))) < eps

    @staticmethod
    def all_equal(a, b):
        """Tensor::all_equal (tensor.rs:330-341)."""
        a = a.numpy() if isinstance(a, Tensor) else np.asarray(a)
        b = b.numpy() if isinstance(b, Tensor) else np.asarray(b)
        return a.shape == b.shape and bool(np.array_equal(a, b))
