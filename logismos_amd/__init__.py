"""logismos_amd -- MI355X (gfx950) ragged-batch decode path for logismos.

The product is the C-ABI shared library ``lib/liblogismos_kernels.so`` built
from ``csrc/`` (declared in ``include/logismos_decode.h``).  The Python modules
here are thin host plumbing over it:

  * ``hip``      -- ctypes view of the HIP runtime (device memory, streams,
                    events), the role `hipcore` plays for the reference;
  * ``kernels``  -- one wrapper per launcher mirroring the reference's
                    ``kernels::launch_*`` (shape guard, then FFI, then status
                    to error).

There is no CPU fallback: a missing library or device raises.
"""
__all__ = ["hip", "kernels"]
