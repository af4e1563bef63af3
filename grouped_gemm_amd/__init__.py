"""Grouped GEMM for AMD Instinct MI355X (gfx950).

Same operator surface as the reference package (grouped_gemm/__init__.py:1-2):
`ops.gmm`, `ops.GroupedGemm`, `backend.gmm`.
"""
from grouped_gemm_amd import backend  # noqa: F401
from grouped_gemm_amd import ops  # noqa: F401
