"""Alternative-implementation names the reference exports from
``cxgnncomp.codegen`` (cxgnncomp/codegen/__init__.py:1-7).  There is no Triton
here: every name runs on the HIP kernels of libcxgnn_hip.so, except
``spmm_torch`` which stays the plain PyTorch sparse product it is upstream."""
from .spmm import spmm_triton, spmm_mm_triton
from .torch_spmm import spmm_torch
from .util import compare, prof, global_res
from .rgcn_kernel import (rgcn_triton, rgcn_triton_opt, rgcn_scatter, rgcn_just_aggr,
                          rgcn_just_aggr_prune, rgcn_full_mm, rgcn_full_mm2, rgcn_prune_mm,
                          rgcn_full_bmm)
from .gen_mapping import Tuner, validate
from .typed_matmul import typed_matmul
from .sddmm import sddmm_dense
