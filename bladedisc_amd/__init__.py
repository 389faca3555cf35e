"""MI355X-native implementation of BladeDISC's quantized-inference hot path.

``libdisc_q8_ral.so`` holds the hand-written gfx950 kernels (int8 MFMA GEMM and
implicit-GEMM convolution with fused requantisation, quantize, dequantize), their
C ABI (include/disc_q8.h) and the RAL runtime they are registered in
(include/tao_ral_api.h).  The Python modules are thin ctypes callers used by the
tests and the benchmark.
"""
__version__ = "0.1.0"
