"""MI355X-native HLQ bit-serial LUT GEMV / small-batch GEMM (drop-in for the
quantized-linear path of Nkniexin/ELUTQ)."""
__version__ = "0.1.0"
