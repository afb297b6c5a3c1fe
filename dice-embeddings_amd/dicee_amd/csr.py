"""Known-answer filter as a CSR.

dicee keeps the filter as ``er_vocab``: a ``defaultdict(list)`` mapping ``(head, relation)`` to the
list of known tails over train+valid+test, duplicates kept
(dicee/read_preprocess_save_load_kg/util.py:355-363, built at preprocess.py:51-60).  The kernels
want, per (head, relation) row, the sorted set of tails: ``row_ptr`` int64 [K+1], ``col`` int32
[nnz], and a way from (h, r) to the row: rows are ordered by the key ``h * num_relations + r``.
"""
import numpy as np
import torch


class FilterCSR:
    def __init__(self, keys, row_ptr, col, num_relations, device=None):
        self._host = (np.ascontiguousarray(keys, dtype=np.int64),       # sorted unique h*R + r
                      np.ascontiguousarray(row_ptr, dtype=np.int64),
                      np.ascontiguousarray(col, dtype=np.int32))
        self.num_relations = int(num_relations)
        self.kind = "er"
        self.device = None
        self.keys = self.row_ptr = self.col = None
        if device is not None:
            self.to(device)

    # ---------------------------------------------------------------- builders
    @classmethod
    def from_triples(cls, triples, num_relations, device=None, max_per_row=None):
        """``triples``: int array [n,3] of (h, r, t); all splits concatenated by the caller."""
        triples = np.asarray(triples)
        h = triples[:, 0].astype(np.int64)
        r = triples[:, 1].astype(np.int64)
        t = triples[:, 2].astype(np.int64)
        key = h * int(num_relations) + r
        order = np.lexsort((t, key))
        key, t = key[order], t[order]
        keep = np.ones(len(key), dtype=bool)
        keep[1:] = (key[1:] != key[:-1]) | (t[1:] != t[:-1])        # drop duplicate (key, t)
        key, t = key[keep], t[keep]
        ukeys, start, counts = np.unique(key, return_index=True, return_counts=True)
        if max_per_row is not None and counts.max(initial=0) > max_per_row:
            pos = np.arange(len(key)) - np.repeat(start, counts)
            sel = pos < max_per_row
            key, t = key[sel], t[sel]
            ukeys, start, counts = np.unique(key, return_index=True, return_counts=True)
        row_ptr = np.zeros(len(ukeys) + 1, dtype=np.int64)
        np.cumsum(counts, out=row_ptr[1:])
        return cls(ukeys, row_ptr, t.astype(np.int32), num_relations, device)

    @classmethod
    def from_triples_gpu(cls, triples, num_entities, num_relations, kind="er"):
        """Build on the GPU (kge_csr_build).  ``triples``: int64 [n,3] GPU tensor of (h, r, t) ids, all splits
        concatenated.  ``kind``: ``"er"`` (h, r) -> tails, the evaluator's filter; ``"re"`` (r, t) -> heads;
        ``"ee"`` (h, t) -> relations.  Out-of-range ids raise ``ValueError``."""
        from . import ops
        N, R = int(num_entities), int(num_relations)
        columns, ranges = {"er": ((0, 1, 2), (N, R, N)), "re": ((1, 2, 0), (R, N, N)),
                           "ee": ((0, 2, 1), (N, N, R))}[kind]
        keys, row_ptr, col, dropped = ops.csr_build(triples.contiguous(), columns, ranges)
        if dropped:
            raise ValueError(f"{dropped} triples hold an id outside [0, {N}) x [0, {R})")
        self = cls.__new__(cls)
        self.num_relations = ranges[1]                                   # multiplier of the key: a * range_b + b
        self.kind = kind
        self.device = triples.device
        self.keys, self.row_ptr, self.col = keys.clone(), row_ptr.clone(), col.clone()
        self._host = None
        return self

    @classmethod
    def from_er_vocab(cls, er_vocab, num_relations, device=None):
        """``er_vocab``: dict (h, r) -> iterable of tails (the reference's structure)."""
        n = sum(len(v) for v in er_vocab.values())
        triples = np.empty((n, 3), dtype=np.int64)
        i = 0
        for (h, r), tails in er_vocab.items():
            m = len(tails)
            triples[i:i + m, 0] = h
            triples[i:i + m, 1] = r
            triples[i:i + m, 2] = np.asarray(tails, dtype=np.int64)
            i += m
        return cls.from_triples(triples, num_relations, device)

    # ---------------------------------------------------------------- access
    def _host_arrays(self):
        if self._host is None:                                           # built on the GPU: mirror on first use
            self._host = (self.keys.cpu().numpy(), self.row_ptr.cpu().numpy(), self.col.cpu().numpy())
        return self._host

    @property
    def keys_np(self):
        return self._host_arrays()[0]

    @property
    def row_ptr_np(self):
        return self._host_arrays()[1]

    @property
    def col_np(self):
        return self._host_arrays()[2]

    def to(self, device):
        device = torch.device(device)
        if self.keys is not None and self.keys.device == device:
            return self
        self.device = device
        self.keys = torch.from_numpy(self.keys_np).to(self.device)
        self.row_ptr = torch.from_numpy(self.row_ptr_np).to(self.device)
        self.col = torch.from_numpy(self.col_np).to(self.device)
        return self

    @property
    def num_rows(self):
        return len(self._host[0]) if self._host is not None else self.keys.numel()

    @property
    def nnz(self):
        return len(self._host[2]) if self._host is not None else self.col.numel()

    def rows_for(self, hr):
        """CSR row of every (h, r) pair of ``hr`` ([B,2] int64 GPU tensor); -1 if unknown (kge_csr_lookup)."""
        from . import ops
        return ops.csr_lookup(hr.contiguous(), self.keys, self.num_relations)

    def rows_for_numpy(self, hr):
        hr = np.asarray(hr, dtype=np.int64)
        key = hr[:, 0] * self.num_relations + hr[:, 1]
        if len(self.keys_np) == 0:
            return np.full(len(key), -1, dtype=np.int64)
        pos = np.searchsorted(self.keys_np, key)
        pos_c = np.minimum(pos, len(self.keys_np) - 1)
        return np.where(self.keys_np[pos_c] == key, pos_c, -1).astype(np.int64)

    def tails(self, h, r):
        """Sorted known tails of (h, r) as a numpy array (empty if the pair is unknown)."""
        row = self.rows_for_numpy(np.array([[h, r]]))[0]
        if row < 0:
            return np.empty(0, dtype=np.int32)
        return self.col_np[self.row_ptr_np[row]:self.row_ptr_np[row + 1]]
