"""ksmm_amd: Kronecker-sparse matrix multiplication for MI355X (gfx950).

``KSLinear(patterns, weights, algo='kernel', dtype, bs_last)`` keeps the reference's API;
``algo='kernel'`` runs hand-written HIP kernels through the C ABI of libksmm_hip.so.
"""
from .layer import (KSLinear, bmm_bs_first, bmm_bs_last, from_abcd_to_dense,  # noqa: F401
                    from_bmm_format_to_dense, from_kernel_format_to_dense, generate_factor,
                    quantize_fp8)
from .kernel import Kernel, query_tile  # noqa: F401
