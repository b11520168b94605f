"""MI355X-native GGUF block-quantized matmul (Ollama's Mulmat hot path) -- Python host side.

``ollama_amd.qmm``  ctypes binding of the C-ABI library ``libmi_qmm.so`` (include/mi_qmm.h).
``ollama_amd.ml``   mirror of the reference's ml.Backend / ml.Context / ml.Tensor interface for this
                    path (/root/reference/ml/backend.go:16-33, 94-128, 130-153).
All compute runs in the HIP library; there is no CPU fallback here.
"""
from . import qmm  # noqa: F401

__all__ = ["qmm", "ml"]
