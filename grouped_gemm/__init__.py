"""Drop-in import name of the reference package: `import grouped_gemm`,
`grouped_gemm.ops.gmm`, `grouped_gemm.backend.gmm` resolve to grouped_gemm_amd
(reference layout: grouped_gemm/__init__.py:1-2)."""
import sys

import grouped_gemm_amd
from grouped_gemm_amd import backend, ops

sys.modules[__name__ + ".ops"] = ops
sys.modules[__name__ + ".backend"] = backend
sys.modules.setdefault("grouped_gemm_backend", backend.backend)
