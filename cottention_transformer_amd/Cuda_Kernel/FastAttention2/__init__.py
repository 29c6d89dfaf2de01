"""`FastAttention2`: the extension module name built by the reference's Cuda_Kernel/setup.py:13
(`CUDAExtension('FastAttention2.kernel', ...)`).  Here it is a Python facade over the C ABI."""
from . import kernel  # noqa: F401
