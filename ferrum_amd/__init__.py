"""MI355X-native quantized matmul for Ferrum's op API (Q4_K / Q6_K GEMV, GEMM, MoE).

``ferrum_amd.api`` mirrors the reference's operator interface over the C ABI
declared in ``include/ferrum_hip.h``; ``ferrum_amd.synth`` builds seeded
synthetic super-blocks.  Importing ``ferrum_amd.api`` fails loudly when the
HIP library has not been built: there is no CPU fallback.
"""
__all__ = ["synth"]
