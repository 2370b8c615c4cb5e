"""A host-side model of the chunked allocator behind sg_ctx_create_pooled, for the tests: the policy of the
reference's Pool (session/memory.rs:199-475) as sage_hip.h states it, on plain integers (chunk id, offset, size).
The branch of the reference it follows is unreachable there (context.rs:49 passes use_cache = false) and the reference
holds no test or vector for it: what the tests pin is that the library follows the stated policy and keeps the
invariants of an allocator, not parity with a run of the reference.
"""
KIB, MIB = 1024, 1024 * 1024
ALIGN = 256
MIN_BLOCK = 512               # memory.rs:23 (x4: the reference counts 4-byte elements)
SMALL_SIZE = 1 * MIB          # memory.rs:25
SMALL_BUFFER = 2 * MIB        # memory.rs:27
LARGE_BUFFER = 20 * MIB       # memory.rs:29
MIN_LARGE = 10 * MIB          # memory.rs:31
ROUND_LARGE = 2 * MIB         # memory.rs:33
SPLIT_LIM = 2 * LARGE_BUFFER  # memory.rs:35


class OutOfMemory(Exception):
    def __init__(self, needed, total):
        super().__init__(f"needed {needed}, total {total}")
        self.needed, self.total = needed, total


class Block:
    def __init__(self, chunk, cap, size, offset):
        self.chunk, self.cap, self.size, self.offset, self.age = chunk, cap, size, offset, 0

    def whole(self):
        return self.size == self.cap


def chunk_size(size):  # allocation_size, memory.rs:257-265
    if size < SMALL_SIZE:
        return SMALL_BUFFER
    if size < MIN_LARGE:
        return LARGE_BUFFER
    return (size + ROUND_LARGE - 1) // ROUND_LARGE * ROUND_LARGE


class Pool:
    def __init__(self, capacity, sub_buffers=True):
        self.capacity, self.sub = capacity, sub_buffers
        self.small, self.large, self.live = [], [], {}
        self.total = self.used = self.peak = 0
        self.next_chunk = 0
        self.chunks_dropped = []  # chunk ids given back to the device, in order

    def _cls(self, size):
        return self.small if size < SMALL_SIZE else self.large

    def _expand(self, size):  # memory.rs:267-283
        n = chunk_size(size)
        if self.capacity and self.total + n > self.capacity:
            raise OutOfMemory(self.total + n - self.capacity, self.total)
        self._cls(size).append(Block(self.next_chunk, n, n, 0))
        self.next_chunk += 1
        self.total += n
        self.peak = max(self.peak, self.total)

    def _take(self, size):  # memory.rs:285-331
        cls = self._cls(size)
        for b in cls:
            b.age += 1
        best = None
        for i, b in enumerate(cls):
            if size > b.size or (not self.sub and not b.whole()):
                continue
            if (size < SPLIT_LIM <= b.size) or (SPLIT_LIM <= size and size + LARGE_BUFFER <= b.size):
                continue
            if best is None or b.size < cls[best].size:
                best = i
        if best is None:
            return None
        b = cls.pop(best)
        b.age = 0
        rest = b.size - size
        if self.sub and ((size <= SMALL_SIZE and MIN_BLOCK <= rest) or (SMALL_SIZE < size < SPLIT_LIM and SMALL_SIZE < rest)):
            cls.append(Block(b.chunk, b.cap, rest, b.offset + size))
            b.size = size
        self.used += b.size
        return b

    def _drop(self, cls, idx):
        for i in sorted(idx, reverse=True):
            b = cls.pop(i)
            self.total -= b.size
        return None

    def _collect(self):  # memory.rs:403-449
        import numpy as np
        if not self.capacity:
            return
        threshold = int(np.float32(self.capacity) * np.float32(0.8))
        if self.used < threshold:
            return
        target = self.capacity - threshold
        ages = [b.age for b in self.large if b.whole()]
        total_age, freeable, reclaimed, freed = sum(ages), len(ages), 0, True
        while reclaimed < target and freed and freeable > 0:
            thr = total_age // freeable
            idx = [i for i, b in enumerate(self.large) if b.whole() and b.age >= thr]
            total_age -= sum(self.large[i].age for i in idx)
            freeable -= len(idx)
            freed = bool(idx)
            reclaimed += sum(self.large[i].size for i in idx)
            self.chunks_dropped += [self.large[i].chunk for i in idx]
            self._drop(self.large, idx)

    def _release(self, size):  # memory.rs:451-475
        released = 0
        while released < max(size, SPLIT_LIM):
            best = None
            for i, b in enumerate(self.large):
                if b.whole() and (best is None or b.size >= self.large[best].size):
                    best = i
            if best is None:
                break
            released += self.large[best].size
            self.chunks_dropped.append(self.large[best].chunk)
            self._drop(self.large, [best])

    def alloc(self, nbytes):  # memory.rs:333-352; returns (chunk id, offset, size)
        size = (max(nbytes, 1) + ALIGN - 1) // ALIGN * ALIGN
        b = self._take(size)
        if b is None:
            self._collect()
            try:
                self._expand(size)
            except OutOfMemory:
                self._release(size)
                try:
                    self._expand(size)
                except OutOfMemory:
                    # the library's addition: whole free chunks of the small class go back as well before it gives up
                    idx = [i for i, b in enumerate(self.small) if b.whole()]
                    if not idx:
                        raise
                    self.chunks_dropped += [self.small[i].chunk for i in idx]
                    self._drop(self.small, idx)
                    self._expand(size)
            b = self._take(size)
            if b is None:
                raise OutOfMemory(size, self.total)
        self.live[(b.chunk, b.offset)] = b
        return b.chunk, b.offset, b.size

    def free(self, key):  # memory.rs:364-396
        b = self.live.pop(key)
        self.used -= b.size
        cls = self.small if b.cap == SMALL_BUFFER else self.large
        b.age = 0
        if self.sub:
            for i in range(len(cls) - 1, -1, -1):
                n = cls[i]
                if n.chunk != b.chunk:
                    continue
                if n.offset + n.size == b.offset:
                    b.offset, b.size = n.offset, b.size + n.size
                    cls.pop(i)
                elif b.offset + b.size == n.offset:
                    b.size += n.size
                    cls.pop(i)
        cls.append(b)

    def trim(self):
        for cls in (self.small, self.large):
            idx = [i for i, b in enumerate(cls) if b.whole()]
            self.chunks_dropped += [cls[i].chunk for i in idx]
            self._drop(cls, idx)
