"""ctypes binding of libag_hip.so (the C ABI declared in include/ag_hip.h).

Nothing here computes: it loads the HIP library, declares the prototypes and turns a non-zero
``ag_status_t`` into a Python exception carrying the library's message.  There is no fallback:
if the library is missing the import of any operator fails loudly.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libag_hip.so")
# The same sources built with -DAG_TEST_HOOKS: the tuning hooks of csrc/ag_test_hooks.h exist only there.
TEST_LIB_PATH = os.path.join(_HERE, "libag_hip_test.so")

c_f = C.c_float
c_i = C.c_int
c_ll = C.c_longlong
c_sz = C.c_size_t
c_p = C.c_void_p


class OpError(RuntimeError):
    """Mirror of the reference's `op::OpError` (src/op.rs:66-73)."""
    code = 0


class NdArrayError(OpError):
    code = 1


class IncompatibleShape(OpError):
    code = 2


class TypeUnsupported(OpError):
    code = 3


class InvalidDims(OpError):
    code = 4


class OutOfBounds(OpError):
    code = 5


class HipError(OpError):
    code = 100


_ERRORS = {1: NdArrayError, 2: IncompatibleShape, 3: TypeUnsupported, 4: InvalidDims, 5: OutOfBounds}

# name -> (restype, argtypes); kept in the order of include/ag_hip.h
PROTOTYPES = {
    "ag_last_error": (C.c_char_p, []),
    "ag_version": (C.c_char_p, []),
    "ag_conv_out_size": (c_i, [c_i] * 5),
    "ag_conv_transpose_out_size": (c_i, [c_i] * 5),
    "ag_pool_out_size": (c_i, [c_i] * 4),
    "ag_pool_grad_in_size": (c_i, [c_i] * 4),
    "ag_im2col_f32": (c_i, [c_p, c_p, c_p] + [c_i] * 12),
    "ag_col2im_f32": (c_i, [c_p, c_p, c_p] + [c_i] * 14),
    "ag_gemm_f32": (c_i, [c_p, c_i, c_i, c_i, c_i, c_i, c_f, c_p, c_i, c_ll, c_p, c_i, c_ll, c_f, c_p,
                          c_i, c_ll, c_i]),
    "ag_gemm_batchsum_f32_workspace": (c_sz, [c_i] * 4),
    "ag_matmul_f32_workspace": (c_sz, [c_i] * 3),
    "ag_matmul_f32": (c_i, [c_p, c_i, c_i, c_i, c_i, c_i, c_p, c_i, c_p, c_i, c_p, c_i, c_p, c_sz]),
    "ag_gemm_batchsum_f32": (c_i, [c_p, c_i, c_i, c_i, c_i, c_i, c_f, c_p, c_i, c_ll, c_p, c_i, c_ll,
                                   c_f, c_p, c_i, c_i, c_p, c_sz]),
    "ag_conv2d_fwd_f32": (c_i, [c_p] * 5 + [c_i] * 10),
    "ag_conv2d_with_cols_f32": (c_i, [c_p] * 4 + [c_i] * 4),
    "ag_conv2d_filter_grad_f32_workspace": (c_sz, [c_i] * 4),
    "ag_conv2d_filter_grad_f32": (c_i, [c_p] * 4 + [c_i] * 4 + [c_p, c_sz]),
    "ag_conv2d_transpose_f32": (c_i, [c_p] * 5 + [c_i] * 12),
    "ag_conv2d_transpose_filter_grad_f32": (c_i, [c_p] * 5 + [c_i] * 12 + [c_p, c_sz]),
    "ag_maxpool2d_fwd_f32": (c_i, [c_p] * 5 + [c_i] * 7),
    "ag_relu_maxpool2d_2x2_f32": (c_i, [c_p] * 8 + [c_i] * 4),
    "ag_maxpool2d_bwd_f32": (c_i, [c_p] * 5 + [c_i] * 7),
    "ag_maxpool2d_bwd_relu_f32": (c_i, [c_p] * 6 + [c_i] * 7),
    "ag_maxpool2d_gradgrad_f32": (c_i, [c_p] * 5 + [c_i] * 7),
    "ag_sum_all_f32_workspace": (c_sz, [c_sz]),
    "ag_sum_all_f32": (c_i, [c_p, c_p, c_sz, c_p, c_p, c_sz]),
    "ag_reduce_sum_f32_workspace": (c_sz, [c_p, c_i, c_p, c_i]),
    "ag_reduce_sum_f32": (c_i, [c_p, c_p, c_p, c_p, c_i, c_p, c_i, c_i, c_p, c_sz]),
    "ag_broadcast_grad_f32": (c_i, [c_p, c_p, c_p, c_p, c_i, c_p, c_i]),
    "ag_adam_update_f32": (c_i, [c_p] * 6 + [c_sz] + [c_f] * 4),
    "ag_adam_update_multi_max": (c_i, []),
    "ag_adam_update_multi_f32": (c_i, [c_p, c_i] + [c_p] * 6 + [c_f] * 4),
    "ag_relu_f32": (c_i, [c_p, c_p, c_p, c_sz]),
    "ag_relu_grad_f32": (c_i, [c_p, c_p, c_p, c_p, c_sz]),
    "ag_add_bias_f32": (c_i, [c_p, c_p, c_p, c_p, c_sz, c_sz]),
    "ag_add_broadcast_f32": (c_i, [c_p, c_p, c_p, c_p, C.POINTER(c_i), C.POINTER(c_i), c_i]),
    "ag_add_broadcast_relu_f32": (c_i, [c_p, c_p, c_p, c_p, C.POINTER(c_i), C.POINTER(c_i), c_i]),
    "ag_bias_grad_f32": (c_i, [c_p, c_p, c_p, c_sz, c_sz]),
    "ag_add_n_f32": (c_i, [c_p, c_p, c_i, c_p, c_sz]),
    "ag_mul_f32": (c_i, [c_p, c_p, c_p, c_p, c_sz]),
    "ag_scale_f32": (c_i, [c_p, c_p, c_f, c_p, c_sz]),
    "ag_div_scalar_f32": (c_i, [c_p, c_p, c_f, c_p, c_sz]),
    "ag_fill_f32": (c_i, [c_p, c_p, c_f, c_sz]),
    "ag_sparse_softmax_xent_f32": (c_i, [c_p] * 5 + [c_sz, c_sz]),
    "ag_sparse_softmax_xent_grad_f32": (c_i, [c_p] * 5 + [c_sz, c_sz]),
    "ag_sparse_softmax_xent_grad_logits_f32": (c_i, [c_p] * 4 + [c_f, c_p, c_sz, c_sz]),
    "ag_conv_input_grad_scratch_floats": (C.c_size_t, [c_i] * 12),
    "ag_conv_input_grad_prepare_f32": (c_i, [c_p, c_p, c_p, c_p] + [c_i] * 12),
    "ag_conv_input_grad_gemm_f32": (c_i, [c_p, c_p, c_p] + [c_i] * 12),
    "ag_conv2d_nocols_scratch_floats": (c_sz, [c_i] * 10),
    "ag_conv2d_fwd_nocols_f32": (c_i, [c_p, c_p, c_p, c_p, c_p] + [c_i] * 10),
    "ag_conv2d_nocols_prepare_f32": (c_i, [c_p, c_p, c_p, c_p] + [c_i] * 10),
    "ag_conv2d_nocols_gemm_f32": (c_i, [c_p, c_p, c_p] + [c_i] * 10),
    "ag_conv2d_nocols_with_filter_f32": (c_i, [c_p, c_p, c_p, c_p, c_p] + [c_i] * 10),
    "ag_conv2d_filter_grad_nocols_f32_workspace": (c_sz, [c_i] * 10),
    "ag_conv2d_filter_grad_nocols_f32": (c_i, [c_p, c_p, c_p, c_p] + [c_i] * 10 + [c_p, c_sz]),
    "ag_matmul_f32_static_scratch_bytes": (c_sz, []),
    "ag_matmul_f32_noalloc": (c_i, [c_p, c_i, c_i, c_i, c_i, c_i, c_p, c_i, c_p, c_i, c_p, c_i]),
}

# Test hooks (csrc/ag_test_hooks.h): thread-local overrides used by the test-suite, not part of the boundary and
# exported by libag_hip_test.so only.
TEST_HOOKS = {
    "ag_test_gemm_force_config": (None, [c_i]),
    "ag_test_gemm_force_splits": (None, [c_i]),
    "ag_test_gemm_force_grid": (None, [c_i]),
    "ag_test_pool_chunk_rows": (None, [c_i]),
}

_lib = None        # what lib() returns: the shipped library, or the test flavour inside use_test_library()
_product = None
_test = None


def _load(path, tables):
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with rust-autograd_amd/csrc/build.sh (there is no CPU fallback)")
    handle = C.CDLL(path)
    for table in tables:
        for name, (res, args) in table.items():
            fn = getattr(handle, name)  # AttributeError names the missing symbol
            fn.restype = res
            fn.argtypes = args
    return handle


def lib():
    """The loaded library.  Raises if it has not been built (run __graft_entry__.build())."""
    global _lib, _product
    if _lib is None:
        if _product is None:
            _product = _load(LIB_PATH, [PROTOTYPES])
        _lib = _product
    return _lib


def test_lib():
    """libag_hip_test.so: the operator boundary plus the hooks of csrc/ag_test_hooks.h."""
    global _test
    if _test is None:
        _test = _load(TEST_LIB_PATH, [PROTOTYPES, TEST_HOOKS])
    return _test


class use_test_library:
    """Context manager: inside it lib() -- and with it every launcher of kernels.py -- is the test flavour of the
    library, so that a test can force tile configurations, split counts and chunk sizes (single-threaded use)."""

    def __enter__(self):
        global _lib
        self.saved = lib()
        _lib = test_lib()
        return _lib

    def __exit__(self, *exc):
        global _lib
        _lib = self.saved
        return False


def last_error():
    return lib().ag_last_error().decode(errors="replace")


def check(status):
    """Raise the exception class that corresponds to a non-zero ag_status_t."""
    if status == 0:
        return
    cls = _ERRORS.get(status, HipError)
    err = cls(last_error())
    err.status = status
    raise err
