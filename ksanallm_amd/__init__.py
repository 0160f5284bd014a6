"""MI355X-native quantized-GEMM subsystem for KsanaLLM's matmul / MoE layers.

The package holds the HIP kernel library (``csrc/`` -> ``libksq_hip.so``, C-ABI in ``include/ksq.h``), its ctypes
binding (:mod:`ksanallm_amd.lib`) and the host-side mirror of the reference's kernel-wrapper functions
(:mod:`ksanallm_amd.ops`).  There is no CPU fallback: importing :mod:`ksanallm_amd.ops` without the built library
raises.
"""
__all__ = ["lib", "ops"]
