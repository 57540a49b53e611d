"""Python restatement of the reference's BFC arena bookkeeping (cuda/bfc.go),
kept structurally literal - a doubly linked free list of memblocks walked the
way the Go code walks it - so that the product's C++ arena can be compared with
it on random alloc/free sequences.  TEST INFRASTRUCTURE ONLY.

Pinned by the reference's own test sequence cuda/bfc_test.go:47-120 (see
tests/test_bfc.py), which fixes addresses and free-list lengths step by step.
"""
from __future__ import annotations

FREE_ALLOC_THRESH = 0.75  # cuda/bfc.go:14


class Memblock:  # cuda/bfc.go:20-34
    __slots__ = ("address", "size", "next", "prev")

    def __init__(self, address, size):
        self.address, self.size, self.next, self.prev = address, size, None, None

    def cap(self):
        return self.address + self.size

    def overlaps(self, b):  # cuda/bfc.go:37-60
        if self is b or self.address == b.address:
            return True
        if self.address < b.address:
            return b.address < self.cap()
        return self.address < b.cap()

    def lt(self, b):  # cuda/bfc.go:76-90
        if self.address == b.address:
            return False
        return self.address < b.address and self.cap() < b.address

    def split(self, size):  # cuda/bfc.go:62-72
        assert size < self.size, "IMPOSSIBLE"
        b = Memblock(self.address + size, self.size - size)
        self.size = size
        return b


class Freelist:  # cuda/bfc.go:96-243
    def __init__(self):
        self.first = self.last = None
        self.l = 0

    def blocks(self):
        out, b = [], self.first
        while b is not None:
            out.append((b.address, b.size))
            b = b.next
        return out

    def insert(self, block):  # cuda/bfc.go:113-219
        if self.first is None:
            self.first = self.last = block
            self.l += 1
            return
        if block.address >= self.last.address:
            if block.overlaps(self.last):
                bc, lc = block.cap(), self.last.cap()
                if bc < lc:
                    return
                self.last.size += bc - lc
                return
            self.last.next = block
            block.prev = self.last
            block.next = None
            self.last = block
            self.l += 1
            return
        if block.address < self.first.address:
            if block.overlaps(self.first):
                bc, fc = block.cap(), self.first.cap()
                if fc < bc:
                    return
                self.first.size += bc - fc
                return
            self.first.prev = block
            block.next = self.first
            self.first = block
            self.l += 1
            return
        b = self.first
        while b is not None:
            ov = b.overlaps(block)
            if b.address < block.address and ov:
                bc, c = block.cap(), b.cap()
                if bc <= c:
                    return
                b.size += c - bc
                return
            if b.address < block.address and not ov:
                if b.next.address >= block.cap():
                    nxt = b.next
                    b.next = block
                    block.next = nxt
                    block.prev = b
                    nxt.prev = block
                    self.l += 1
                    return
            elif b.address == block.address:
                if b.size > block.size:
                    return
                b.size = block.size
                return
            elif b.address > block.address and ov:
                bc, c = block.cap(), b.cap()
                b.address = block.address
                b.size = block.size if c <= bc else block.size + (c - bc)
                return
            elif b.address > block.address and not ov:
                break
            b = b.next
        raise AssertionError("Unreachable")

    def remove(self, block):  # cuda/bfc.go:221-240
        if self.first is block:
            self.first = block.next
        else:
            block.prev.next = block.next
        if self.last is block:
            self.last = block.prev
        else:
            block.next.prev = block.prev
        block.next = block.prev = None
        self.l -= 1

    def split_or_remove(self, block, aligned, size):  # cuda/bfc.go:243-256
        if block.size > aligned:
            self.insert(block.split(aligned))
        if block.size > size:
            self.insert(block.split(size))
        self.remove(block)


class OOM(Exception):
    def __init__(self, res, allocated):
        super().__init__(f"allocated/reserved: {allocated}/{res}")  # cuda/errors.go:13
        self.res, self.allocated = res, allocated


class BFCOracle:  # cuda/bfc.go:298-467
    def __init__(self, alignment):
        self.block_size = alignment
        self.freelist = Freelist()
        self.used = {}
        self.start = self.size = self.reserved = 0
        self.allocated = self.allocs = self.frees = 0

    def reserve(self, start, size):
        self.start = start
        self.size = size - (size % self.block_size)
        self.reserved = size
        self.freelist.insert(Memblock(0, size))

    def align(self, size):
        rem = size % self.block_size
        return size if rem == 0 else size - rem + self.block_size

    def best_fit(self, size):
        b = self.freelist.first
        while b is not None:
            if b.size >= size:
                return b
            b = b.next
        return None

    def alloc(self, size):
        if size <= 0:
            raise ValueError("Cannot allocate memory with size 0 or less")
        aligned = self.align(size)
        block = self.best_fit(aligned)
        if block is None:
            self.coalesce()
            block = self.best_fit(aligned)
            if block is None:
                raise OOM(self.size, self.allocated)
        self.freelist.split_or_remove(block, aligned, size)
        self.used[block.address] = size
        self.allocated += size
        self.allocs += 1
        return block.address + self.start

    def free(self, address):
        a = address - self.start
        if a not in self.used:
            return
        size = self.used.pop(a)
        self.freelist.insert(Memblock(a, size))
        self.allocated -= size
        self.frees += 1
        if self.frees / self.allocs >= FREE_ALLOC_THRESH:
            self.coalesce()

    def coalesce(self):
        block = self.freelist.first
        while block is not None:
            if block.address % self.block_size == 0:
                nxt = block.next
                while nxt is not None:
                    if block.cap() == nxt.address:
                        block.size += nxt.size
                        block.next = nxt.next
                        if nxt.next is not None:
                            # the Go code leaves next.next.prev stale; remove() only reads
                            # prev of the block being removed, so keep the list consistent
                            nxt.next.prev = block
                        if nxt is self.freelist.last:
                            self.freelist.last = block
                        self.freelist.l -= 1
                        nxt = block.next
                    elif block.overlaps(nxt):
                        raise AssertionError("Unhandled: overlapping coalesceing")
                    else:
                        break
            block = block.next

    def reset_allocator(self):  # cuda/arena.go:25-36
        for k in list(self.used):
            self.free(k + self.start)
        self.coalesce()
        self.allocated = self.allocs = self.frees = 0
