"""``Batch``: the container a sampled mini-batch travels in, with the reference's
raw little-endian ``.dat`` layout on disk (cxgnncomp/batch.py:7-90): ``ptr.dat`` and
``idx.dat`` as int64, ``x.dat`` / ``y.dat`` as written by numpy ``tofile``, sizes in
``num_node_in_layer.dat`` / ``num_edge_in_layer.dat`` (int64)."""
import os

import numpy as np
import torch


class Batch:

    def __init__(self, x, ptr, idx, num_node_in_layer, num_edge_in_layer=None, y=None, edge_index=None):
        self.x = x
        self.ptr = ptr
        self.idx = idx
        self.y = y
        self.edge_index = edge_index
        self.num_node_in_layer = num_node_in_layer
        self.num_edge_in_layer = num_edge_in_layer

    def to(self, device):
        for name in ("x", "ptr", "idx", "y", "edge_index"):
            v = getattr(self, name)
            if isinstance(v, torch.Tensor):
                setattr(self, name, v.to(device))
        return self

    def tofile(self, path):
        os.makedirs(path, exist_ok=True)
        for name in ("x", "ptr", "idx", "y"):
            v = getattr(self, name)
            if isinstance(v, torch.Tensor):
                v.detach().cpu().numpy().tofile(os.path.join(path, name + ".dat"))
        for name in ("num_node_in_layer", "num_edge_in_layer"):
            v = getattr(self, name)
            if v is not None:
                np.asarray(torch.as_tensor(v).cpu(), dtype=np.int64).tofile(os.path.join(path, name + ".dat"))

    @staticmethod
    def fromfile(path, feat_len, device="cpu", x_dtype=np.float32):
        def load(name, dtype):
            p = os.path.join(path, name + ".dat")
            return torch.from_numpy(np.fromfile(p, dtype=dtype)) if os.path.exists(p) else None
        x = load("x", x_dtype)
        if x is not None:
            x = x.reshape(-1, feat_len)
        nn = load("num_node_in_layer", np.int64)
        ne = load("num_edge_in_layer", np.int64)
        b = Batch(x, load("ptr", np.int64), load("idx", np.int64), nn, ne, load("y", np.int64))
        return b.to(device)


PyGBatch = Batch
