"""`sgl_kernel` as the reference's callers import it (sgl-kernel/python/sgl_kernel/__init__.py):
the operators of the W8A8 quantized-linear path, served by the gfx950 library in `sglang_amd`.
Importing it registers the torch.ops.sgl_kernel.* entries of the path."""

from sglang_amd.sgl_kernel import *  # noqa: F401,F403
from sglang_amd.sgl_kernel import __all__  # noqa: F401
