"""Same five public names as the reference's ``self_ops/ops_py/__init__.py:1-12``."""
from .approx_ops import (approx_conv2d_baseline_op, approx_conv2d_op, approx_gemm_baseline_op, approx_gemm_op,
                         init_lookup_tables)

__all__ = ["init_lookup_tables", "approx_gemm_op", "approx_gemm_baseline_op", "approx_conv2d_op",
           "approx_conv2d_baseline_op"]
