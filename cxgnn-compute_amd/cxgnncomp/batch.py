"""``Batch`` and ``PyGBatch``: the containers a mini-batch travels in
(cxgnncomp/batch.py:7-90), with the reference's raw ``.dat`` layout on disk:
``x.dat`` (float32), ``ptr.dat`` / ``idx.dat`` / ``target.dat`` (int64), each the flat
little-endian image numpy ``tofile`` writes.

Same constructor arguments, attributes and methods as the reference class.  Two things are
added, none changed: ``tofile`` also writes ``num_node_in_layer.dat`` /
``num_edge_in_layer.dat`` (int64; the reference keeps the layer sizes outside the files), and
``Batch.load`` reads a directory back into a ready batch (features reshaped, sizes restored).
``todgl`` needs DGL, which is not part of this package, and raises.
"""
import os

import numpy as np
import torch


def _read(path, dtype):
    return torch.from_numpy(np.fromfile(path, dtype=dtype))


class Batch:

    def __init__(self, x, ptr, idx, num_node_in_layer=None, num_edge_in_layer=None, target=None,
                 edge_index=None):
        self.x = x
        self.ptr = ptr
        self.idx = idx
        self.num_node_in_layer = num_node_in_layer
        self.num_edge_in_layer = num_edge_in_layer
        self.target = target
        self.block = None
        self.edge_index = edge_index

    def to(self, dev):
        """Moves the tensors in place (cxgnncomp/batch.py:26-36); returns self for chaining."""
        for name in ("x", "ptr", "idx", "target", "edge_index", "block"):
            v = getattr(self, name, None)
            if v is not None and hasattr(v, "to"):
                setattr(self, name, v.to(dev))
        return self

    def tofile(self, dir):
        os.makedirs(dir, exist_ok=True)
        for name in ("x", "ptr", "idx", "target"):
            v = getattr(self, name)
            if v is not None:
                v.detach().cpu().numpy().tofile(os.path.join(dir, name + ".dat"))
        for name in ("num_node_in_layer", "num_edge_in_layer"):
            v = getattr(self, name)
            if v is not None:
                np.asarray(torch.as_tensor(v).cpu(), dtype=np.int64).tofile(os.path.join(dir, name + ".dat"))

    def fromfile(self, dir):
        """Fills this batch from the files of ``dir`` (cxgnncomp/batch.py:48-62): every tensor comes
        back flat, ``x`` included, exactly as the reference leaves it."""
        for name, dtype in (("x", np.float32), ("ptr", np.int64), ("idx", np.int64), ("target", np.int64)):
            path = os.path.join(dir, name + ".dat")
            if os.path.exists(path):
                setattr(self, name, _read(path, dtype))
            elif name == "ptr":
                print(path, "not found")

    @classmethod
    def load(cls, dir, feat_len, device="cpu"):
        """A batch read back from ``dir``: ``fromfile`` plus ``x`` reshaped to [*, feat_len] and the
        layer sizes, if their files are there."""
        b = cls(None, None, None)
        b.fromfile(dir)
        if b.x is not None:
            b.x = b.x.reshape(-1, feat_len)
        for name in ("num_node_in_layer", "num_edge_in_layer"):
            path = os.path.join(dir, name + ".dat")
            if os.path.exists(path):
                setattr(b, name, _read(path, np.int64))
        return b.to(device)

    def todgl(self, num_src, num_dst):
        raise NotImplementedError("Batch.todgl builds a DGL block (cxgnncomp/batch.py:64-77); DGL is not "
                                  "part of this package, which runs the CSR graph types")

    def totype(self, dtype):
        self.ptr = self.ptr.to(dtype)
        self.idx = self.idx.to(dtype)
        self.target = self.target.to(dtype)


class PyGBatch:
    """Features plus a COO ``edge_index`` (cxgnncomp/batch.py:86-90)."""

    def __init__(self, x, edge_index):
        self.x = x
        self.edge_index = edge_index
