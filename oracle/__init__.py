"""CPU oracle for the depthwise conv2d path -- TEST INFRASTRUCTURE ONLY.

Two independent checkers live here:

* ``dwconv_oracle.c`` (loaded through ctypes): a double-precision closed-form
  restatement of the reference's four kernels
  (torch_dwconv/dwconv_kernel.cu:69-181, :260-306, :308-442, :444-588).
* ``torch_reference``: ``F.conv2d(groups=C)`` in fp64 on the CPU plus autograd,
  which is the oracle the reference's own tests use (test/test_forward.py:14)
  and the function the reference itself falls back to (torch_dwconv/dwconv.py:126-128).

``host_logic`` restates the reference's pure-Python argument handling
(torch_dwconv/dwconv.py:39-44, :76-130).

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  The shipped package never does.
"""
from .capi import (  # noqa: F401
    build,
    out_size,
    use_dwconv2d_small,
    dwconv2d,
    dwconv2d_small,
    backward_kernel,
    forward,
    grad_input,
    grad_weight,
)
from .torch_reference import (  # noqa: F401
    torch_reference,
    torch_reference_fused,
    torch_reference_general,
    torch_cpu_fp32_step,
    shift_add_reference,
)
from . import host_logic  # noqa: F401
