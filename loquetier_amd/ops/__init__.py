"""Operator namespace mirroring `loquetier.ops` for the SMLM path.

A reference checkout switches to these kernels by replacing
`from loquetier.ops import _kernels as kernel`
(src/loquetier_src/kernel_utils.py:8) with
`from loquetier_amd.ops import _kernels as kernel`.
"""
from . import _kernels  # noqa: F401
