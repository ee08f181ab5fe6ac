"""Restatement of the reference's KV-cache cell bookkeeping (test infrastructure: only tests may import this).

llama_kv_cache keeps, per cell, a position and a set of sequence ids, and a ring position `head` where the search for free
cells starts.  Each function follows the reference function named in its docstring; the cells' tensors are not modelled, only
the metadata that decides where a step's rows go and what each token may attend.
"""
import numpy as np


class KvCells:
    def __init__(self, size):
        self.size = size
        self.pos = [-1] * size          # llama_kv_cell (llama.cpp:1381-1390)
        self.seq = [set() for _ in range(size)]
        self.head = 0
        self.n = 0

    def find_slot(self, positions, seq_ids):
        """llama_kv_cache_find_slot, llama.cpp:1683-1730.  seq_ids[i]: list of ids of token i.  Returns False when no run is free."""
        n_ctx, n_tokens = self.size, len(positions)
        if n_tokens > n_ctx:
            return False
        n_tested = 0
        while True:
            if self.head + n_tokens > n_ctx:
                n_tested += n_ctx - self.head
                self.head = 0
                continue
            found = True
            for i in range(n_tokens):
                if self.pos[self.head + i] >= 0:
                    found = False
                    self.head += i + 1
                    n_tested += i + 1
                    break
            if found:
                break
            if n_tested >= n_ctx:
                return False
        for i in range(n_tokens):
            self.pos[self.head + i] = int(positions[i])
            for s in seq_ids[i]:
                self.seq[self.head + i].add(int(s))
        return True

    def cell_max(self):
        """llama_kv_cache_cell_max, llama.cpp:1735-1743 (cell 0 alone counts as 0, as there)."""
        for i in range(self.size - 1, 0, -1):
            if self.pos[i] >= 0 and self.seq[i]:
                return i + 1
        return 0

    def decode(self, positions, seq_ids):
        """The cache's part of llama_decode_internal, llama.cpp:6834-6842 and 6936-6943: slot, the cell range of the step, the mask of
        :6506-6531 ([n_tokens][n] floats, 0 or -inf), then the head moves past the step.  Returns (first cell, n, mask) or None."""
        if not self.find_slot(positions, seq_ids):
            return None
        first = self.head
        self.n = min(self.size, max(32, self.cell_max()))
        mask = np.zeros((len(positions), self.n), np.float32)
        for j in range(len(positions)):
            for i in range(self.n):
                if seq_ids[j][0] not in self.seq[i] or self.pos[i] > positions[j]:
                    mask[j, i] = -np.inf
        self.head += len(positions)
        if self.head >= self.size:
            self.head = 0
        return first, self.n, mask

    def seq_rm(self, seq_id, p0, p1):
        """llama_kv_cache_seq_rm, llama.cpp:1757-1785"""
        new_head = self.size
        if p0 < 0:
            p0 = 0
        if p1 < 0:
            p1 = 2 ** 31 - 1
        for i in range(self.size):
            if p0 <= self.pos[i] < p1:
                if seq_id < 0:
                    self.seq[i].clear()
                elif seq_id in self.seq[i]:
                    self.seq[i].discard(seq_id)
                else:
                    continue
                if not self.seq[i]:
                    self.pos[i] = -1
                    if new_head == self.size:
                        new_head = i
        if new_head != self.size:
            self.head = new_head

    def seq_cp(self, src, dst, p0, p1):
        """llama_kv_cache_seq_cp, llama.cpp:1787-1803"""
        if p0 < 0:
            p0 = 0
        if p1 < 0:
            p1 = 2 ** 31 - 1
        self.head = 0
        for i in range(self.size):
            if src in self.seq[i] and p0 <= self.pos[i] < p1:
                self.seq[i].add(dst)

    def seq_keep(self, seq_id):
        """llama_kv_cache_seq_keep, llama.cpp:1805-1822"""
        new_head = self.size
        for i in range(self.size):
            if seq_id not in self.seq[i]:
                self.pos[i] = -1
                self.seq[i].clear()
                if new_head == self.size:
                    new_head = i
            else:
                self.seq[i] = {seq_id}
        if new_head != self.size:
            self.head = new_head

    def clear(self):
        """llama_kv_cache_clear, llama.cpp:1745-1751"""
        self.pos = [-1] * self.size
        self.seq = [set() for _ in range(self.size)]
        self.head = 0

    def state(self):
        bits = np.array([sum(1 << s for s in c) for c in self.seq], np.uint32)
        return np.array(self.pos, np.int32), bits, self.head
