"""MI355X-native graph kernels behind the CxGNN-Compute Python API.

Hot-path names of the reference package (cxgnncomp/__init__.py:1-18) are
importable from here; everything runs on libcxgnn_hip.so through
``cxgnncomp_backend``.
"""
from . import synthetic  # noqa: F401
