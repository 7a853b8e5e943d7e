"""Drop-in for the reference's pybind module ``cxgnncomp_backend``
(src/cpp/python_bindings/binding.cpp:14-130), backed by libcxgnn_hip.so.

Same function names, argument order and meaning.  Differences, all deliberate:
  * errors raise ValueError / RuntimeError instead of exit(1)
    (src/cpp/include/common.h:16-26);
  * the nine launch integers of the ``*_configurable`` functions are accepted
    and ignored -- the HIP kernels balance work by edge spans themselves;
  * gradients w.r.t. node features are computed by gathering over a cached
    transposed CSR instead of fp32 atomics, so they are deterministic;
  * the autograd contexts keep the ptr/idx tensors alive instead of raw
    pointers (src/cpp/src/aggr.cu:116-117).
"""
import torch

from . import _lib, _ops
from ._ops import as_int, clear_graph_cache, set_graph_cache_capacity  # noqa: F401


def _lib_version():
    return _lib.load().cxg_version()


# --------------------------------------------------------------------------- #
# Aggregation, SDDMM and edge-attention families: the compiled host layer
# (csrc_ext/backend_ext.cpp), under the reference's names and argument order.
#   run_spmm_configurable / _bwd / _int32     src/cpp/src/spmm_host.cu:6-156   (binding.cpp:37-41)
#   sage_sum_forward / sage_mean_forward / sage_*_forward_edge_value
#                                             src/cpp/src/aggr.cu:107-303,377-393 -- autograd in C++
#   spmm_multihead / _bwd / run_spmm_multihead_configurable, SPMM_MULTIHEAD_SCHEDULE
#                                             src/cpp/src/spmm_host.cu:158-256 (binding.cpp:57-74)
#   run_sddmm / run_sddmm_vertex_centric      src/cpp/src/sddmm_host.cu:4-59   (binding.cpp:76-79)
#   edge_attention(ptr, idx, att_dst, att_src, num_edge, relu_l) -- dst before src --,
#   edge_value_degree, spmv                   src/cpp/src/edge_softmax.cu:97-244 -- autograd in C++
# The nine launch integers of the *_configurable functions are accepted and ignored.
# --------------------------------------------------------------------------- #
_C = _lib.native()

run_spmm_configurable = _C.run_spmm_configurable
run_spmm_configurable_int32 = _C.run_spmm_configurable_int32
run_spmm_configurable_bwd = _C.run_spmm_configurable_bwd
sage_sum_forward = _C.sage_sum_forward
sage_mean_forward = _C.sage_mean_forward
sage_sum_forward_edge_value = _C.sage_sum_forward_edge_value
sage_mean_forward_edge_value = _C.sage_mean_forward_edge_value      # raises, as the reference aborts (aggr.cu:158,163)

SPMM_MULTIHEAD_SCHEDULE = _C.SPMM_MULTIHEAD_SCHEDULE
Naive, PreReduce, Optimal = _C.Naive, _C.PreReduce, _C.Optimal
spmm_multihead = _C.spmm_multihead
spmm_multihead_bwd = _C.spmm_multihead_bwd
run_spmm_multihead_configurable = _C.run_spmm_multihead_configurable

run_sddmm = _C.run_sddmm
run_sddmm_vertex_centric = _C.run_sddmm_vertex_centric

edge_attention = _C.edge_attention
edge_value_degree = _C.edge_value_degree
spmv = _C.spmv


# gather(input[E, F], dest[E], num_node): out[dest[e]] += input[e] (src/cpp/src/aggr.cu:395-448,
# binding.cpp:19); autograd in C++, destination groups cached per destination array
gather = _C.gather

from ._rel import (aggr_rel, selective_aggr, selective_aggr_bwd, target_aggr,  # noqa: E402,F401
                   target_aggr_backward)
from ._typed import (aggr_rel_direct, aggr_rgcn_direct_func, aggr_rgcn_mean, pad_rel, pad_rel_idx,  # noqa: E402,F401
                     seastar_backward, seastar_forward, typed_linear, typed_linear_s2d,
                     typed_linear_s2e)
from ._schedule import (COMPUTEOP, REDUCEOP, GSpMM_u, GSpMM_u_e, gen_edge_type_mag240m,  # noqa: E402,F401
                        rel_schedule, topo_sort)

SUM, MAX, MIN, MEAN = REDUCEOP.SUM, REDUCEOP.MAX, REDUCEOP.MIN, REDUCEOP.MEAN
ADD, MUL, DIV, SUB = COMPUTEOP.ADD, COMPUTEOP.MUL, COMPUTEOP.DIV, COMPUTEOP.SUB
