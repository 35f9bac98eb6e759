"""loquetier_amd: MI355X-native Segmented Multi-LoRA Multiplication (SMLM).

Only the SMLM path of Loquetier lives here: the HIP kernels and their C ABI
(csrc/, include/smlm.h) and the Python operator surface the reference's LoRA
layer calls (ops/_kernels.py, kernel_utils.py, mixed_lora.py, segments.py).
"""
__version__ = "0.1.0"
