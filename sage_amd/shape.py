"""Stride algebra of tensors: the host-side mirror of the reference's `Shape` (shape.rs).

Pure integer arithmetic, no device involved.  Every method cites the reference method it mirrors;
the semantics (including the quirks: `insert` gives stride 0, `has_default_strides` ignores the
offset) are the reference's, because the kernels' fast paths are chosen from exactly these values.
"""


class ShapeError(ValueError):
    """shape.rs:12-35 ShapeError."""


def default_strides(extents):
    """Shape::default_strides (shape.rs:45-54)."""
    size = 1
    for e in extents:
        size *= e
    out = []
    for e in extents:
        size //= e if e else 1
        out.append(size)
    return out


def union(s1, s2):
    """shape::union (shape.rs:356-393): right-aligned NumPy-style broadcast of two extents."""
    s1, s2 = list(s1), list(s2)
    if s1 == s2:
        return s1
    longer, shorter = (s1, s2) if len(s1) > len(s2) else (s2, s1)
    u = longer[:len(longer) - len(shorter)] + shorter
    for i, (a, b) in enumerate(zip(u, longer)):
        if a != b:
            if a == 1:
                u[i] = b
            elif b != 1:
                raise ShapeError("invalid broadcast")
    return u


def norm_axis(axis, bound):
    """Axis::to_usize (shape.rs:480-520): negative axes count from the end."""
    a = axis + bound if axis < 0 else axis
    if not 0 <= a < bound:
        raise ShapeError("invalid index bound")
    return a


def norm_axes(axes, bound):
    if isinstance(axes, int):
        axes = [axes]
    return [norm_axis(int(a), bound) for a in axes]


def infer_extents(extents, size):
    """Extent::to_arr (shape.rs:540-640): `size` 0 means "not specified"; one entry may be -1 and is
    then inferred from `size`; any other non-positive entry is invalid; a specified size must match."""
    extents = [int(e) for e in extents]
    for e in extents:
        if e < 1 and e != -1:
            raise ShapeError(f"invalid extent {e}")
    n_infer = extents.count(-1)
    if n_infer > 1:
        raise ShapeError("invalid inference")
    known = 1
    for e in extents:
        if e != -1:
            known *= e
    if n_infer == 1:
        if size == 0 or size % known:
            raise ShapeError("invalid inference")
        extents[extents.index(-1)] = size // known
    elif size != 0 and known != size:
        raise ShapeError(f"size mismatch ({size}, {known})")
    return extents


class Shape:
    """extents / strides (in elements) / offset (in elements)  — shape.rs:38-42."""

    __slots__ = ("extents", "strides", "offset")

    def __init__(self, extents, strides=None, offset=0):
        self.extents = [int(e) for e in extents]
        self.strides = default_strides(self.extents) if strides is None else [int(s) for s in strides]
        self.offset = int(offset)
        if len(self.extents) != len(self.strides):
            raise ShapeError("extents and strides differ in length")

    def __eq__(self, other):
        return (isinstance(other, Shape) and self.extents == other.extents
                and self.strides == other.strides and self.offset == other.offset)

    def __repr__(self):
        return f"Shape(extents={self.extents}, strides={self.strides}, offset={self.offset})"

    def copy(self):
        return Shape(self.extents, self.strides, self.offset)

    @property
    def rank(self):
        return len(self.extents)

    def size(self):
        n = 1
        for e in self.extents:
            n *= e
        return n

    def translate_default(self, index):
        """shape.rs:89-100: linear index in default order -> element index in the buffer."""
        out = self.offset
        p = self.size()
        rem = index
        for e, s in zip(self.extents, self.strides):
            p //= e
            c = rem // p
            rem -= c * p
            out += c * s
        return out

    def extract(self, axes, nested):
        """shape.rs:113-132: (inner = listed axes in listed order, outer = the rest)."""
        inner = Shape([self.extents[a] for a in axes], [self.strides[a] for a in axes], 0 if nested else self.offset)
        rest = [a for a in range(self.rank) if a not in axes]
        outer = Shape([self.extents[a] for a in rest], [self.strides[a] for a in rest], self.offset)
        return inner, outer

    def has_default_strides(self):
        """shape.rs:134-143 (the offset is not looked at)."""
        return self.strides == default_strides(self.extents)

    def is_contiguous(self):
        """shape.rs:148-168."""
        max_index = sum((e - 1) * s for e, s in zip(self.extents, self.strides))
        t = 1
        for e, s in zip(self.extents, self.strides):
            if s > 0:
                t *= e
        return max_index == t - 1

    def is_bijective(self):
        """shape.rs:172-174."""
        return all(s > 0 for s in self.strides)

    def remove(self, axis):
        """shape.rs:183-188."""
        s = self.copy()
        del s.extents[axis], s.strides[axis]
        return s

    def insert(self, axis):
        """shape.rs:190-195: extent 1 with stride 0."""
        s = self.copy()
        s.extents.insert(axis, 1)
        s.strides.insert(axis, 0)
        return s

    def swap(self, a1, a2):
        """shape.rs:197-202."""
        s = self.copy()
        s.extents[a1], s.extents[a2] = s.extents[a2], s.extents[a1]
        s.strides[a1], s.strides[a2] = s.strides[a2], s.strides[a1]
        return s

    def permute(self, axes):
        """shape.rs:204-215."""
        return Shape([self.extents[a] for a in axes], [self.strides[a] for a in axes], self.offset)

    def select(self, index, axis):
        """shape.rs:217-228."""
        if self.rank <= axis:
            raise ShapeError("axis out of bounds")
        if self.extents[axis] <= index:
            raise ShapeError("index out of bounds")
        s = self.copy()
        s.offset += s.strides[axis] * index
        return s.remove(axis)

    def select_range(self, start, end, axis):
        """shape.rs:230-237: inclusive end."""
        if self.extents[axis] <= end:
            raise ShapeError("index out of bounds")
        s = self.copy()
        s.offset += self.strides[axis] * start
        s.extents[axis] = end - start + 1
        return s

    def reshape_view(self, extents):
        """Strides that present this (possibly non-dense) layout with `extents` without moving data,
        or None when no such strides exist.  The reference always copies a non-default layout before
        a reshape (core.rs:213-233); this is the zero-copy case analysis it skips: old axes are
        grouped into runs that are contiguous among themselves and each run is re-split."""
        extents = [int(e) for e in extents]
        n = 1
        for e in extents:
            n *= e
        if n != self.size():
            return None
        old = [(e, s) for e, s in zip(self.extents, self.strides) if e != 1]
        new_strides = [0] * len(extents)
        oi = 0
        ni = 0
        while ni < len(extents):
            if extents[ni] == 1:
                new_strides[ni] = 0
                ni += 1
                continue
            if oi >= len(old):
                return None
            # take old axes until their product covers a run of new axes
            op, np_ = old[oi][0], extents[ni]
            o_start, n_start = oi, ni
            while op != np_:
                if op < np_:
                    oi += 1
                    if oi >= len(old):
                        return None
                    op *= old[oi][0]
                else:
                    ni += 1
                    if ni >= len(extents):
                        return None
                    np_ *= extents[ni]
            # the old axes of this run must be contiguous among themselves
            for k in range(o_start, oi):
                if old[k][1] != old[k + 1][1] * old[k + 1][0]:
                    return None
            stride = old[oi][1]
            for k in range(ni, n_start - 1, -1):
                new_strides[k] = stride
                stride *= extents[k]
            oi += 1
            ni += 1
        if oi != len(old):
            return None
        return Shape(extents, new_strides, self.offset)

    def expand(self, extents):
        """shape.rs:239-279: left-pad with (1, stride 0), then mute broadcast axes with stride 0."""
        extents = [int(e) for e in extents]
        if len(extents) < self.rank:
            raise ShapeError("target shape must be larger than the broadcasted shape")
        ne, ns = list(self.extents), list(self.strides)
        for _ in range(len(extents) - self.rank):
            ne.insert(0, 1)
            ns.insert(0, 0)
        for i, e in enumerate(extents):
            if ne[i] != e:
                if ne[i] == 1:
                    ne[i], ns[i] = e, 0
                else:
                    raise ShapeError("invalid broadcast... target shape should be larger.")
        return Shape(ne, ns, self.offset)
