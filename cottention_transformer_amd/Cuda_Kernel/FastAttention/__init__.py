"""`FastAttention`: the older extension of the reference -- sub-modules `forward` and `backward`
(Cuda_Kernel/setup.py:7-12) plus the flat names of Cuda_Kernel/pybind.cpp:10-27."""
from . import backward, forward  # noqa: F401

forward_float32, forward_float16, forward_bfloat16 = forward.float32, forward.float16, forward.bfloat16
backward_float32, backward_float16, backward_bfloat16 = backward.float32, backward.float16, backward.bfloat16
