"""MI355X-native graph kernels behind the CxGNN-Compute Python API.

The hot-path names of the reference package (cxgnncomp/__init__.py:1-18) are
importable from here and run on libcxgnn_hip.so through ``cxgnncomp_backend``.
The model stacks (``SAGE``, ``GCN``, ``GIN``, ``GAT``, ``RGCN``) run the CSR graph types;
trainer and dataset loading of the reference need dgl / PyG / cxgnndl and are not part of
this package.
"""
from .graph_conv import (MyGATConv, MyGCNConv, MySageConv, MyGINConv, MyRGCNConv, RGCNOP, RGCNOP2,
                         RGCNOP3, RGCNOP_sorted, AggrOP, AggrDirectedOP, SeastarRGCNOP, run_rgcn4)
from cxgnncomp_backend import (edge_attention, sage_sum_forward_edge_value, gather, sage_sum_forward,
                               aggr_rel, sage_mean_forward, aggr_rel_direct, rel_schedule, target_aggr)
from .codegen import *  # noqa: F401,F403
from .timer import TimerOP, TimerModule, Timers, set_timers, get_timers
from .typed_linear import (TypedLinearE2EOP, TypedLinearS2EOP, TypedLinearS2DMMAggrOP,
                           TypedLinearS2DAggrMMOP, TypedLinearS2DSort, TypedLinearNaiveS2D,
                           TypedLinearS2DPushOP, SelectMMS2EOP)
from .schedule import (neighbor_grouping, neighbor_grouping_gpu, partition_2d, reorder_by,
                       remove_from_graph, remove_from_graph_by_edge)
from .batch import Batch, PyGBatch
from .util import global_tuner
from .graph_kernel import SpMMValOP
from .batchnorm import BatchNorm1d
from .model import (GNN, SAGE, GCN, GIN, GAT, RGCN, get_model, get_conv_from_str, get_model_from_str,
                    graph_type_dict, model_dict)
from . import synthetic  # noqa: F401
