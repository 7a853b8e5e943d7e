"""Layer stacks of the reference's model zoo on the HIP backend
(cxgnncomp/model.py:16-287): ``GNN`` and its ``SAGE`` / ``GCN`` / ``GIN`` / ``GAT`` /
``RGCN`` specialisations for the two CSR graph types.

  * graph_type "CSR": one full graph per batch, every layer aggregates all rows of ``ptr``;
  * graph_type "CSR_Layer": a sampled mini-batch in one nested CSR, layer i of an
    L-layer model aggregates rows [0, num_node_in_layer[L-1-i]) over the edge prefix
    idx[:num_edge_in_layer[L-1-i]] (model.py:55-71).

Between layers: BatchNorm1d, ReLU, dropout; the output is ``log_softmax``.  The DGL /
PyG graph types of the reference need those packages and raise here.
"""
import torch
import torch.nn.functional as F

import cxgnncomp_backend

from .batchnorm import BatchNorm1d
from .graph_conv import MyGATConv, MyGCNConv, MyGINConv, MyRGCNConv, MySageConv


def _need_csr(graph_type):
    if "CSR" not in graph_type:
        raise NotImplementedError("graph type %r needs DGL / PyG; this package runs the CSR graph types"
                                  % (graph_type,))


class GNN(torch.nn.Module):

    def __init__(self, in_channels, hidden_channels, out_channels, num_layer, dropout, graph_type,
                 config=None, **kwargs):
        super().__init__()
        _need_csr(graph_type)
        self.in_channels = in_channels
        self.hidden_channels = hidden_channels
        self.out_channels = out_channels
        self.graph_type = graph_type
        self.num_layer = num_layer
        self.dropout = dropout
        self.bns = torch.nn.ModuleList(BatchNorm1d(hidden_channels) for _ in range(num_layer - 1))
        self.init_convs(**kwargs)

    def init_convs(self, **kwargs):
        widths = [self.in_channels] + [self.hidden_channels] * (self.num_layer - 1)
        outs = [self.hidden_channels] * (self.num_layer - 1) + [self.out_channels]
        if self.num_layer == 1:                      # upstream builds in -> hidden only (model.py:33-35)
            outs = [self.hidden_channels]
        self.convs = torch.nn.ModuleList(
            self.init_conv(widths[i], outs[i], layer=i, **kwargs) for i in range(self.num_layer))

    def init_conv(self, in_channels, out_channels, **kwargs):
        raise NotImplementedError

    def reset_parameters(self):
        for m in list(self.convs) + list(self.bns):
            m.reset_parameters()

    # rows / edges layer i works on
    def _rows(self, batch, i):
        if self.graph_type == "CSR_Layer":
            return int(batch.num_node_in_layer[self.num_layer - 1 - i])
        # upstream passes 0 (= "all rows" for the sage_* ops only, src/cpp/src/aggr.cu:118);
        # the explicit row count means the same there and also suits the other layers
        return batch.ptr.shape[0] - 1

    def _between(self, x, i):
        x = self.bns[i](x, relu=True)              # = F.relu(bn(x)), upstream model.py:66-67
        return F.dropout(x, p=self.dropout, training=self.training)

    def layer(self, conv, x, batch, i):
        return conv(x, batch.ptr, batch.idx, self._rows(batch, i))

    def forward_cxg(self, batch, skip_first=False):
        x = batch.x
        sizes = (getattr(batch, "num_node_in_layer", None), getattr(batch, "num_edge_in_layer", None))
        if (self.graph_type == "CSR_Layer" and batch.ptr.is_cuda and sizes[0] is not None and sizes[1] is not None
                and not any(getattr(v, "is_cuda", False) for v in sizes) and len(sizes[1]) + 1 == len(sizes[0])):
            # the batch knows its layers' edge counts: the backward passes then build the reversed
            # graphs without waiting for the device to report ptr[num_node] per layer
            cxgnncomp_backend._ops.note_edge_counts(batch.ptr, batch.idx, batch.num_node_in_layer[:-1],
                                                    batch.num_edge_in_layer)
        last = self.num_layer - 1
        for i, conv in enumerate(self.convs):
            if not (skip_first and i == 0 and i != last):
                x = self.layer(conv, x, batch, i)
            if i != last:
                x = self._between(x, i)
        return x.log_softmax(dim=-1)

    def forward(self, input, skip_first=False):
        _need_csr(self.graph_type)
        return self.forward_cxg(input)


class SAGE(GNN):

    def init_conv(self, in_channels, out_channels, **kwargs):
        return MySageConv(in_channels, out_channels)


class GCN(GNN):

    def init_conv(self, in_channels, out_channels, **kwargs):
        return MyGCNConv(in_channels, out_channels)


class GIN(GNN):

    def init_conv(self, in_channels, out_channels, **kwargs):
        return MyGINConv(in_channels, out_channels)


class GAT(GNN):

    def init_conv(self, in_channels, out_channels, **kwargs):
        kwargs = dict(kwargs)
        if "heads" in kwargs and out_channels % kwargs["heads"] != 0:
            kwargs["heads"] = 1
        if kwargs.get("concat"):
            out_channels = out_channels // kwargs.get("heads", 1)
        return MyGATConv(in_channels, out_channels, **kwargs)

    def layer(self, conv, x, batch, i):
        assert self.graph_type == "CSR_Layer"
        k = self.num_layer - 1 - i
        return conv(x, batch.ptr, batch.idx, num_dst=int(batch.num_node_in_layer[k]),
                    num_src=int(batch.num_node_in_layer[k + 1]), num_edge=int(batch.num_edge_in_layer[k]))

    def forward_cxg(self, batch, skip_first=False):
        return super().forward_cxg(batch, False)


class RGCN(GNN):

    def init_conv(self, in_channels, out_channels, **kwargs):
        self.num_rel = kwargs["num_rel"]
        self.dataset_name = kwargs.get("dataset_name", "")
        self.gen_rel = self.dataset_name == "rmag240m"
        if self.gen_rel:
            self.num_rel = 5
        return MyRGCNConv(in_channels, out_channels, num_rel=self.num_rel)

    def edge_types(self, batch):
        """Relation of every edge: from the global node ids for MAG240M, else the batch's own
        ``etypes`` when it carries them, else uniform random as upstream (model.py:172-177)."""
        if self.gen_rel:
            return cxgnncomp_backend.gen_edge_type_mag240m(batch.ptr, batch.idx, batch.sub_to_full)
        if getattr(batch, "etypes", None) is not None:
            return batch.etypes
        n = int(batch.num_edge_in_layer[self.num_layer - 1]) if self.graph_type == "CSR_Layer" \
            else batch.idx.shape[0]
        return torch.randint(0, self.num_rel, (n,), device=batch.x.device)

    def forward_cxg(self, batch, skip_first=False):
        self._etypes = self.edge_types(batch)
        return super().forward_cxg(batch, False)

    def layer(self, conv, x, batch, i):
        et = self._etypes
        if self.graph_type == "CSR_Layer":
            et = et[:int(batch.num_edge_in_layer[self.num_layer - 1 - i])]
        return conv(x, batch.ptr, batch.idx, et, self._rows(batch, i))


# --------------------------------------------------------------------------- #
# Factories (cxgnncomp/model.py:345-467)
# --------------------------------------------------------------------------- #
graph_type_dict = {
    "cxg": "CSR_Layer",
    "dgl": "DGL",
    "pyg": "PyG",
}

model_dict = {
    "gcn": GCN,
    "gat": GAT,
    "gin": GIN,
    "rgcn": RGCN,
    "sage": SAGE,
}


def _item(node, key, default=None):
    """``node[key]`` / ``node.key`` of a config node (omegaconf, dict or plain namespace)."""
    if isinstance(node, dict):
        return node.get(key, default)
    getter = getattr(node, "get", None)
    if callable(getter):
        try:
            return getter(key, default)
        except TypeError:
            pass
    return getattr(node, key, default)


def get_model(config):
    """Model from a training configuration (cxgnncomp/model.py:362-399): reads
    ``dl.dataset.{feature_dim, num_classes, name}``, ``dl.sampler.train.num_layer``,
    ``train.type`` (cxg / dgl / pyg) and ``train.model.{type, hidden_dim, dropout, heads, concat,
    num_rel}``.  The dgl / pyg graph types raise NotImplementedError."""
    dataset = config.dl.dataset
    spec = config.train.model
    kind = str(_item(spec, "type")).lower()
    graph_type = graph_type_dict[str(config.train.type).lower()]
    args = (_item(dataset, "feature_dim"), _item(spec, "hidden_dim"), _item(dataset, "num_classes"),
            config.dl.sampler.train.num_layer, _item(spec, "dropout"), graph_type, config)
    if "gat" in kind:
        return model_dict[kind](*args, heads=_item(spec, "heads", 1), concat=_item(spec, "concat", False))
    if "rgcn" in kind:
        return model_dict[kind](*args, num_rel=int(_item(spec, "num_rel")),
                                dataset_name=str(_item(dataset, "name")).lower())
    return model_dict[kind](*args)


def get_conv_from_str(model_str, infeat, outfeat, num_head=-1, num_rel=-1):
    """One convolution layer by name (cxgnncomp/model.py:402-414)."""
    model_str = model_str.lower()
    if model_str == "gat":
        return MyGATConv(infeat, outfeat, heads=num_head)
    if model_str == "gcn":
        return MyGCNConv(infeat, outfeat)
    if model_str == "sage":
        return MySageConv(infeat, outfeat)
    if model_str == "rgcn":
        return MyRGCNConv(infeat, outfeat, num_rel=num_rel)
    assert False, f"unknown model {model_str}"


def get_model_from_str(mtype, infeat, hiddenfeat, outfeat, graph_type, num_layer, num_head=-1, num_rel=-1,
                       dataset=None, dropout=0.5):
    """One layer stack by name (cxgnncomp/model.py:417-467).  ``LSTM`` (the neighbour-LSTM
    aggregator) is outside this package."""
    mtype = mtype.upper()
    common = dict(dropout=dropout, graph_type=graph_type, config=None)
    if mtype == "GCN":
        return GCN(infeat, hiddenfeat, outfeat, num_layer, **common)
    if mtype == "GAT":
        return GAT(infeat, hiddenfeat, outfeat, num_layer, heads=num_head, **common)
    if mtype == "SAGE":
        return SAGE(infeat, hiddenfeat, outfeat, num_layer, **common)
    if mtype == "RGCN":
        return RGCN(infeat, hiddenfeat, outfeat, num_layer, num_rel=num_rel, dataset_name=dataset, **common)
    if mtype == "GIN":
        return GIN(infeat, hiddenfeat, outfeat, num_layer, **common)
    if mtype == "LSTM":
        raise NotImplementedError("the neighbour-LSTM model (cxgnncomp/neighbor_lstm.py) is not part of this package")
    assert False, f"unknown model {mtype}"
