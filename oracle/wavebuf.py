"""Wave-buffer bookkeeping and copies, restated with plain Python lists.

LruModel follows BufferManager in
library/retroinfer/retroinfer_kernels/src/wave_buffer_cpu.cpp (:190-257 access, :102-188
update); the copy functions are the loop oracles of
library/retroinfer/test/test_gather_copy.py (:110-127, :190-194, :233-237).
Block ids: the reference takes them from an unordered_set (iteration order unspecified,
:153-156); this model hands out the lowest free id last released first, like the library.
DeviceLruModel restates the device-side manager: the same policy, kept as (step, order in step) pairs.
"""
import torch


class LruModel:
    def __init__(self, sizes, block, capacity, buffer_size):
        self.block, self.capacity, self.buffer_size = block, capacity, buffer_size
        self.sizes = [int(s) for s in sizes]
        self.start = []
        row = 0
        for s in self.sizes:
            self.start.append(row)
            row += s
        self.nblk = [(s + block - 1) // block for s in self.sizes]
        self.resident = {}          # cluster -> list of block ids
        self.lru = []               # most recent first
        self.free = list(range(capacity - 1, -1, -1))  # stack, pops 0,1,2,...
        self.hit_keys, self.miss_keys = [], []
        self.overflow = 0

    def _blocks(self, c):
        n = self.nblk[c]
        out = []
        for j in range(n):
            last = self.sizes[c] - (n - 1) * self.block
            out.append(self.block if j < n - 1 else last)
        return out

    def access(self, ids):
        hit, miss = [], []   # entries (src index, size, cumsum)
        self.hit_keys, self.miss_keys = [], []
        pages = hs = ms = 0
        for c in ids:
            c = int(c)
            pages += self.nblk[c]
            if pages > self.buffer_size:
                self.overflow += 1
                break
            if self.nblk[c] == 0:
                continue
            if c in self.resident:
                self.hit_keys.append(c)
                for bid, sz in zip(self.resident[c], self._blocks(c)):
                    hit.append((bid, sz, hs)); hs += sz
            else:
                self.miss_keys.append(c)
                row = self.start[c]
                for sz in self._blocks(c):
                    miss.append((row, sz, ms)); ms += sz; row += self.block
        return hit, miss

    def update(self):
        for c in reversed(self.hit_keys):
            self.lru.remove(c); self.lru.insert(0, c)
        admit, need = 0, 0
        for c in self.miss_keys:
            if need + self.nblk[c] > self.capacity:
                break
            need += self.nblk[c]; admit += 1
        upd = []   # (cache block id, size, buffer offset)
        if admit:
            while len(self.free) < need and self.lru:
                v = self.lru.pop()
                for b in reversed(self.resident.pop(v)):
                    self.free.append(b)
            off = 0
            for c in self.miss_keys[:admit]:
                ids = []
                for sz in self._blocks(c):
                    b = self.free.pop(); ids.append(b)
                    upd.append((b, sz, off)); off += sz
                self.resident[c] = ids
                self.lru.insert(0, c)
        self.hit_keys, self.miss_keys = [], []
        return upd



class DeviceLruModel:
    """The device-side manager (csrc/lru.hip), one group, plain Python: the reference's policy (LruModel) with
    the manager's own bookkeeping.  Recency is a pair per resident cluster instead of a linked list: the number
    of the last step that touched it and its order inside that step, which reproduces the list of
    wave_buffer_cpu.cpp:106-114 and :170-176 (hits are moved to the front in reverse rank order, then the
    admitted misses are pushed in rank order): inside a step the admitted misses are more recent than the hits,
    later-ranked misses more recent than earlier ones, earlier-ranked hits more recent than later ones.
    Victims are taken from the least recent end until the request is covered, hits of the current step included
    (:140-142).  Freed block ids are appended to the free list in ascending cluster id; admitted clusters take
    ids off the end of the list in rank order (block id VALUES are the manager's own: the reference takes them
    from an unordered_set)."""

    def __init__(self, sizes, block, capacity, buffer_size, stage_row0=None):
        self.block, self.capacity, self.buffer_size = block, capacity, buffer_size
        self.stage_row0 = stage_row0           # set: also keep the row table for attention in place
        self.rows = []
        self.sizes = [int(s) for s in sizes]
        self.start, row = [], 0
        for s_ in self.sizes:
            self.start.append(row)
            row += s_
        self.nblk = [(s_ + block - 1) // block for s_ in self.sizes]
        self.stamp = [0] * len(self.sizes)     # 0: not resident, else the step of the last touch
        self.sub = [0] * len(self.sizes)       # order inside that step (larger = more recent)
        self.blocks = {}                       # resident cluster -> block ids
        self.free = list(range(capacity))
        self.epoch = 0

    def _blocks(self, c):
        n = self.nblk[c]
        return [self.block] * (n - 1) + [self.sizes[c] - (n - 1) * self.block] if n else []

    def step(self, ids):
        """Returns (hit, miss, update) lists of (index, size, offset) triples like LruModel."""
        E = self.epoch + 1
        hit, miss, hits, misses = [], [], [], []
        pages = hs = ms = 0
        self.rows = []
        for c in ids:
            c = int(c)
            if c < 0 or c >= len(self.sizes):
                continue
            pages += self.nblk[c]
            if pages > self.buffer_size:
                break
            if self.nblk[c] == 0:
                continue
            if self.stamp[c] != 0:
                hits.append(c)
                for bid, sz in zip(self.blocks[c], self._blocks(c)):
                    hit.append((bid, sz, hs)); hs += sz
                    self.rows += [bid * self.block + i for i in range(sz)]
            else:
                misses.append((c, ms))
                if self.stage_row0 is not None:
                    self.rows += [self.stage_row0 + ms + i for i in range(self.sizes[c])]
                row = self.start[c]
                for sz in self._blocks(c):
                    miss.append((row, sz, ms)); ms += sz; row += self.block
        for i, c in enumerate(hits):
            self.stamp[c] = E
            self.sub[c] = len(hits) - 1 - i
        admit, need = [], 0
        for c, off in misses:
            if need + self.nblk[c] > self.capacity:
                break
            need += self.nblk[c]; admit.append((c, off))
        to_free = need - len(self.free)
        if to_free > 0:
            order = sorted(self.blocks, key=lambda c: (self.stamp[c], self.sub[c]))   # least recent first
            victims, got = [], 0
            for c in order:
                if got >= to_free:
                    break
                victims.append(c); got += self.nblk[c]
            for c in sorted(victims):
                self.free.extend(self.blocks.pop(c))
                self.stamp[c] = 0
        F = len(self.free)
        upd, taken = [], 0
        for j, (c, off) in enumerate(admit):
            ids_c = [self.free[F - 1 - (taken + k)] for k in range(self.nblk[c])]
            for k, (b, sz) in enumerate(zip(ids_c, self._blocks(c))):
                upd.append((b, sz, off + k * self.block))
            self.blocks[c] = ids_c
            self.stamp[c] = E
            self.sub[c] = len(hits) + j
            taken += self.nblk[c]
        del self.free[F - taken:]
        self.epoch = E
        return hit, miss, upd

def gather_copy_vectors(src_k, src_v, src_m, idx, copy_start, copy_num):
    """test_gather_copy.py:233-237."""
    sel = idx[:, copy_start:copy_start + copy_num]
    g = torch.arange(src_k.shape[0])[:, None]
    return src_k[g, sel], src_v[g, sel], src_m[g, sel]


def concat_gather(dst_k, dst_v, k1, v1, k2, v2, k3, v3, off2, sz2, num2, off3, sz3, num3, copy1):
    """test_gather_copy.py:110-127 (in place on dst_*); returns valid lengths."""
    G = dst_k.shape[0]
    valid = []
    for i in range(G):
        dst_k[i, :copy1] = k1[i, :copy1]; dst_v[i, :copy1] = v1[i, :copy1]
        n = copy1
        for j in range(int(num2[i])):
            s, o = int(sz2[i, j]), int(off2[i, j])
            dst_k[i, n:n + s] = k2[i, o:o + s]; dst_v[i, n:n + s] = v2[i, o:o + s]; n += s
        for j in range(int(num3[i])):
            s, b = int(sz3[i, j]), int(off3[i, j])
            dst_k[i, n:n + s] = k3[i, b, :s]; dst_v[i, n:n + s] = v3[i, b, :s]; n += s
        valid.append(n)
    return valid


def gather_scatter(cache_k, cache_v, src_k, src_v, src_off, sizes, dst_block, num, start):
    """test_gather_copy.py:190-194 (in place on cache_*)."""
    for i in range(cache_k.shape[0]):
        for j in range(int(num[i])):
            s, o, b = int(sizes[i, j]), int(src_off[i, j]), int(dst_block[i, j])
            cache_k[i, b, :s] = src_k[i, start + o:start + o + s]
            cache_v[i, b, :s] = src_v[i, start + o:start + o + s]
