"""MI355X (gfx950) implementation of rust-autograd's conv / matmul / pool / reduce / Adam path.

The product is `libag_hip.so` (sources in csrc/, C ABI in include/ag_hip.h).  The Python modules
here are plumbing around it: `capi` binds the C ABI with ctypes, `kernels` allocates outputs as
torch CUDA tensors and launches.  The directory name contains a hyphen, so it is loaded with
`__graft_entry__.load_package()` under the module name `rust_autograd_amd`.
"""
from . import capi  # noqa: F401
