"""Drop-in for the third-party `grouped_gemm` package (fanshiqing/grouped_gemm v1.1.4) that the
reference binds at moe/grouped_gemm_util.py:3-22: `grouped_gemm.ops.gmm` and `grouped_gemm.backend.gmm`
on the gfx950 persistent grouped-GEMM kernel."""
from . import backend, ops  # noqa: F401
