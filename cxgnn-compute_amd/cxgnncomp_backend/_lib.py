"""ctypes loader for libcxgnn_hip.so (the C ABI declared in include/cxgnn_hip.h).

The library is built in-tree by ``build.py`` next to this package.  Nothing here
falls back to another implementation: if the shared object is missing or a call
fails, a RuntimeError is raised.
"""
import ctypes
import os

import torch  # noqa: F401  (loads the HIP runtime the library links against)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.normpath(os.path.join(_HERE, "..", "lib", "libcxgnn_hip.so"))

_c = ctypes
_P = _c.c_void_p
_I64 = _c.c_int64
_I32 = _c.c_int
_U32 = _c.c_uint
_SZ = _c.c_size_t
_F32 = _c.c_float

# name -> (restype, argtypes); mirrors include/cxgnn_hip.h one to one.
SIGNATURES = {
    "cxg_version": (_I32, []),
    "cxg_last_error": (_c.c_char_p, []),
    "cxg_spmm_workspace_bytes": (_SZ, [_I64, _I64]),
    "cxg_spmm_sum_f32": (_I32, [_P, _P, _P, _I64, _P, _I64, _I64, _I64, _I32, _U32, _P, _SZ, _P]),
    "cxg_spmm_sum_f32_noalloc": (_I32, [_P, _P, _P, _I64, _P, _I64, _I64, _I64, _I32, _U32, _P]),
    "cxg_spmm_sum_f32_i32": (_I32, [_P, _P, _P, _I64, _P, _I64, _I64, _I64, _I32, _U32, _P, _SZ, _P]),
    "cxg_spmm_weighted_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _I32, _I32,
                                     _U32, _P, _SZ, _P]),
    "cxg_spmm_weighted_heads_f32": (_I32, [_P, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _I32, _I32, _U32, _P, _SZ, _P]),
    "cxg_spmm_bf16_rows": (_I32, [_P, _P, _P, _P, _P, _I64, _I32, _P, _I64, _I32, _I64, _I64, _I32, _U32, _P, _SZ, _P]),
    "cxg_spmm_prereduce_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _P, _I64, _I64, _I64, _I32, _I32,
                                      _U32, _P, _SZ, _P]),
    "cxg_spmm_weighted_bias_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _P, _P, _I64, _I64, _I64, _I32, _I32,
                                          _U32, _P, _SZ, _P]),
    "cxg_spmm_weighted_dot_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _P, _I64, _P, _I64, _P, _I64, _I64, _I32, _I32,
                                         _U32, _P, _SZ, _P]),
    "cxg_spmm_ext_f32": (_I32, [_P, _P, _P, _I64, _P, _I64, _I64, _I64, _I32, _U32, _P, _P, _P, _I64,
                                _P, _P, _P, _SZ, _P]),
    "cxg_spmm_scatter_atomic_f32": (_I32, [_P, _P, _P, _I64, _P, _P, _P, _P, _I64, _I64, _I32, _P]),
    "cxg_typed_gemm_f32": (_I32, [_P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I32, _I32, _I32, _U32, _P]),
    "cxg_typed_gemm_epilogue_f32": (_I32, [_P, _I64, _P, _P, _P, _I64, _P, _I64, _P, _P, _P, _I64, _I32, _I32, _I32,
                                            _U32, _P]),
    "cxg_typed_gemm_bf16": (_I32, [_P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I32, _I32, _I32, _U32, _P]),
    "cxg_typed_gemm_wide_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "cxg_typed_gemm_wide_f32": (_I32, [_P, _I64, _P, _P, _I64, _P, _P, _P, _I64, _I32, _I32, _I32, _U32, _P, _SZ, _P]),
    "cxg_rel_segment_workspace_bytes": (_SZ, [_I64, _I32, _I32]),
    "cxg_rel_segment_i64": (_I32, [_P, _I64, _I32, _P, _P, _P, _SZ, _P]),
    "cxg_rel_segment_i32": (_I32, [_P, _I64, _I32, _P, _P, _P, _SZ, _P]),
    "cxg_sddmm_csr_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _P]),
    "cxg_sddmm_coo_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _I32, _I32, _I32, _P]),
    "cxg_edge_softmax_fwd_f32": (_I32, [_P, _P, _P, _P, _P, _P, _I64, _I32, _F32, _P]),
    "cxg_edge_softmax_bwd_f32": (_I32, [_P, _P, _P, _P, _P, _P, _I64, _I32, _F32, _P]),
    "cxg_edge_softmax_bwd_at_f32": (_I32, [_P, _P, _P, _P, _P, _P, _P, _I64, _I32, _F32, _P]),
    "cxg_narrow_gather_sum_f32": (_I32, [_P, _P, _P, _P, _I64, _I32, _P]),
    "cxg_scatter_add_rows_f32": (_I32, [_P, _P, _P, _I64, _I32, _P]),
    "cxg_gather_rows_f32": (_I32, [_P, _P, _P, _I64, _I32, _P]),
    "cxg_head_sum_f32": (_I32, [_P, _P, _I64, _I32, _I32, _P]),
    "cxg_csr_transpose_workspace_bytes": (_SZ, [_I64, _I64]),
    "cxg_csr_transpose_i64": (_I32, [_P, _P, _I64, _I64, _I64, _P, _P, _P, _P, _SZ, _P]),
    "cxg_csr_transpose_prefix_workspace_bytes": (_SZ, [_I64]),
    "cxg_csr_transpose_prefix_i64": (_I32, [_P, _P, _P, _I64, _I64, _I64, _P, _P, _P, _P, _SZ, _P]),
    "cxg_csr_row_ids_i64": (_I32, [_P, _I64, _I64, _P, _P]),
    "cxg_edge_value_degree_f32": (_I32, [_P, _I64, _P, _P]),
    "cxg_pad_rel_i64": (_I32, [_P, _P, _P, _I32, _I32, _I64, _P]),
    "cxg_typed_gemm_wgrad_workspace_bytes": (_SZ, [_I64, _I32, _I32, _I32]),
    "cxg_typed_gemm_wgrad_f32": (_I32, [_P, _I64, _P, _I64, _P, _P, _P, _I64, _I32, _I32, _I32, _P, _U32, _P, _SZ,
                                        _P]),
    "cxg_csr_row_ids_i32": (_I32, [_P, _I64, _I64, _P, _P]),
    "cxg_segment_gather_sum_workspace_bytes": (_SZ, [_I64, _I32]),
    "cxg_segment_gather_sum_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _I64, _I32, _P, _SZ, _P]),
    "cxg_gspmm_workspace_bytes": (_SZ, [_I64, _I32]),
    "cxg_gspmm_i32_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _I64, _I32, _I32, _I32, _P, _SZ, _P]),
    "cxg_topo_sort_host_i64": (_I64, [_P, _P, _P, _I64, _P]),
    "cxg_scan_workspace_bytes": (_SZ, [_I64]),
    "cxg_neighbor_group_plan_i64": (_I32, [_P, _I64, _I64, _P, _P, _SZ, _P]),
    "cxg_neighbor_group_fill_i64": (_I32, [_P, _P, _I64, _I64, _I64, _P, _P, _P]),
    "cxg_filter_rows_plan_i64": (_I32, [_P, _I64, _P, _P, _P, _P, _SZ, _P]),
    "cxg_filter_rows_fill_i64": (_I32, [_P, _P, _I64, _P, _P, _I64, _P, _P, _P]),
    "cxg_filter_edges_plan_i64": (_I32, [_P, _I64, _I64, _P, _P, _I32, _P, _P, _P, _SZ, _P]),
    "cxg_filter_edges_fill_i64": (_I32, [_P, _P, _I64, _I64, _P, _P, _P, _P, _P, _P]),
    "cxg_coo_to_csr_workspace_bytes": (_SZ, [_I64, _I64]),
    "cxg_coo_to_csr_i64": (_I32, [_P, _P, _I64, _I64, _P, _P, _P, _P, _SZ, _P]),
    "cxg_attention_logits_fwd_f32": (_I32, [_P, _P, _P, _I64, _I64, _I32, _I32, _P, _P, _P]),
    "cxg_attention_logits_workspace_bytes": (_SZ, [_I64, _I32, _I32]),
    "cxg_attention_logits_bwd_f32": (_I32, [_P, _P, _P, _P, _P, _I64, _I64, _I32, _I32, _P, _I32, _P, _P, _P, _SZ,
                                            _P]),
    "cxg_attention_logits_proj_supported": (_I32, [_I32, _I32]),
    "cxg_attention_logits_proj_fwd_f32": (_I32, [_P, _I64, _P, _I64, _I64, _I32, _I32, _P, _P, _P]),
    "cxg_attention_logits_proj_workspace_bytes": (_SZ, [_I32, _I32]),
    "cxg_attention_logits_proj_bwd_f32": (_I32, [_P, _I64, _P, _P, _P, _I64, _I64, _I32, _I32, _P, _I64, _I32, _P,
                                                _P, _SZ, _P]),
    "cxg_batchnorm_workspace_bytes": (_SZ, [_I64, _I32]),
    "cxg_column_sum_f32": (_I32, [_P, _I64, _I32, _I64, _P, _P, _SZ, _P]),
    "cxg_batchnorm_stats_f32": (_I32, [_P, _I64, _I32, _I64, _F32, _P, _P, _P, _P, _SZ, _P]),
    "cxg_batchnorm_apply_f32": (_I32, [_P, _I64, _I32, _I64, _P, _P, _P, _P, _P, _I64, _I32, _P]),
    "cxg_batchnorm_bwd_f32": (_I32, [_P, _P, _I64, _I32, _I64, _I64, _P, _P, _P, _P, _I32, _P, _I64, _P, _P, _P,
                                     _SZ, _P]),
}

_lib = None


def load():
    """Return the loaded library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libcxgnn_hip.so not found at %s; build it with `python build.py` in %s"
            % (LIB_PATH, os.path.dirname(os.path.dirname(LIB_PATH))))
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


_native_mod = None


def native():
    """The compiled host layer ``cxgnncomp_backend._C`` (csrc_ext/backend_ext.cpp, built by
    ``build.py``): tensor checks, allocation, the transposed-graph cache and the autograd functions
    of the aggregation family in C++.  Like the library itself it has no substitute."""
    global _native_mod
    if _native_mod is None:
        load()                         # resolves libcxgnn_hip.so, which the extension links against
        try:
            from . import _C
        except ImportError as exc:
            raise RuntimeError("the compiled host layer cxgnncomp_backend/_C.so is missing or does not load (%s); "
                               "build it with `python build.py` in %s"
                               % (exc, os.path.dirname(os.path.dirname(LIB_PATH)))) from exc
        _native_mod = _C
    return _native_mod


def check(status):
    if status != 0:
        msg = load().cxg_last_error().decode("utf-8", "replace")
        if status == -1:
            raise ValueError("cxgnn_hip: " + msg)
        raise RuntimeError("cxgnn_hip (status %d): %s" % (status, msg))


def ptr(t):
    """Device address of a tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


def current_stream(device):
    return torch.cuda.current_stream(device).cuda_stream
