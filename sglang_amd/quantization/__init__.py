"""Callers' glue of the W8A8 path (quantize -> GEMM -> bias), mirroring
python/sglang/srt/layers/quantization/{fp8_kernel,int8_kernel,fp8_utils,w8a8_int8}.py."""
