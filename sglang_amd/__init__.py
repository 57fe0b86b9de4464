"""MI355X (gfx950) kernels for SGLang's W8A8 quantized-linear path.

``sglang_amd.sgl_kernel`` carries the operator names and signatures of the
reference's ``sgl_kernel`` package for this path; ``sglang_amd.quantization``
carries the callers' glue (quantize -> GEMM -> bias)."""

__version__ = "0.1.0"
