"""CPU-side checks of the C-ABI library: it loads without a GPU, exports every function that
include/ag_hip.h declares, the ctypes prototypes cover the header, and the host-only helpers and
argument validation behave like the reference (no kernel is launched here)."""
import ctypes as C
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def capi():
    import __graft_entry__ as entry
    pkg = entry.load_package()
    if not os.path.exists(pkg.capi.LIB_PATH):
        subprocess.check_call(["bash", os.path.join(entry.PKG_DIR, "csrc", "build.sh")])
    return pkg.capi


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "ag_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ag_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_operator_surface():
    names = _declared_functions()
    for needed in ("ag_im2col_f32", "ag_col2im_f32", "ag_gemm_f32", "ag_conv2d_fwd_f32",
                   "ag_conv2d_filter_grad_f32", "ag_conv2d_transpose_f32",
                   "ag_conv2d_transpose_filter_grad_f32", "ag_maxpool2d_fwd_f32", "ag_maxpool2d_bwd_f32",
                   "ag_sum_all_f32", "ag_reduce_sum_f32", "ag_adam_update_f32"):
        assert needed in names


def test_library_exports_every_declared_symbol(capi):
    handle = C.CDLL(capi.LIB_PATH)
    for name in _declared_functions():
        assert hasattr(handle, name), f"{name} is declared in ag_hip.h but not exported"


def test_ctypes_prototypes_cover_the_header(capi):
    assert sorted(capi.PROTOTYPES) == _declared_functions()
    capi.lib()


def _exported(path):
    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True).stdout
    return sorted(l.split()[-1] for l in out.splitlines() if " T " in l and l.split()[-1].startswith("ag_"))


def test_shipped_library_exports_exactly_the_header(capi):
    """libag_hip.so exports the functions of include/ag_hip.h and nothing else: no test or tuning hook."""
    assert _exported(capi.LIB_PATH) == sorted(_declared_functions())
    assert not [n for n in _declared_functions() if n.startswith("ag_test_")]


def test_test_flavour_exports_the_header_plus_the_hooks(capi):
    """libag_hip_test.so (the same sources with -DAG_TEST_HOOKS) adds the thread-local hooks of
    csrc/ag_test_hooks.h, which the public header does not declare."""
    hooks_h = open(os.path.join(ROOT, "rust-autograd_amd", "csrc", "ag_test_hooks.h")).read()
    hooks_h = re.sub(r"/\*.*?\*/", "", hooks_h, flags=re.S)
    hooks = sorted(set(re.findall(r"\b(ag_test_[a-z0-9_]+)\s*\(", hooks_h)))
    assert hooks == sorted(capi.TEST_HOOKS)
    assert _exported(capi.TEST_LIB_PATH) == sorted(_declared_functions() + hooks)
    capi.test_lib()  # loads, and every prototype and hook resolves


def test_library_has_gfx950_code_object(capi):
    blob = open(capi.LIB_PATH, "rb").read()
    assert b"gfx950" in blob
    assert capi.lib().ag_version() == b"ag_hip 0.1.0 gfx950"


def test_library_does_not_link_the_oracle(capi):
    out = subprocess.run(["ldd", capi.LIB_PATH], capture_output=True, text=True).stdout
    assert "oracle" not in out
    assert b"orc_" not in open(capi.LIB_PATH, "rb").read()


def test_geometry_helpers_match_reference_formulas(capi):
    L = capi.lib()
    assert L.ag_conv_out_size(56, 3, 1, 1, 1) == 56
    assert L.ag_conv_out_size(56, 3, 1, 2, 1) == 28
    assert L.ag_conv_out_size(14, 3, 2, 1, 2) == 14
    assert L.ag_conv_out_size(5, 3, 1, 2, 1) == 3
    # conv2d_transpose.rs:55-56: 2*(28-1) - 2 + 3 = 55, one short of the true 56
    assert L.ag_conv_transpose_out_size(28, 3, 1, 2, 1) == 55
    assert L.ag_conv_transpose_out_size(14, 4, 1, 2, 1) == 28
    assert L.ag_pool_out_size(56, 3, 0, 2) == 27
    assert L.ag_pool_out_size(28, 2, 0, 2) == 14
    # max_pool2d.rs:263-264: 2*(27-1) + 3 = 55
    assert L.ag_pool_grad_in_size(27, 3, 0, 2) == 55


def test_validation_errors_map_to_op_error_variants(capi):
    """Argument checks run on the host before anything is launched."""
    L = capi.lib()
    null = C.c_void_p(0)
    # pooling with pad != 0 is outside the reference's defined domain -> InvalidDims
    st = L.ag_maxpool2d_fwd_f32(null, null, null, null, null, 1, 1, 4, 4, 2, 1, 2)
    assert st == 4 and b"pad must be 0" in L.ag_last_error()
    with pytest.raises(capi.InvalidDims):
        capi.check(st)
    # stride 0
    st = L.ag_im2col_f32(null, null, null, 1, 1, 4, 4, 3, 3, 0, 0, 0, 1, 1, 1)
    assert st == 4
    # leading dimension too small -> IncompatibleShape
    st = L.ag_gemm_f32(null, 0, 0, 4, 4, 4, 1.0, null, 2, 0, null, 4, 0, 0.0, null, 4, 0, 1)
    assert st == 2 and b"lda" in L.ag_last_error()
    # axis out of range -> OutOfBounds
    shape = (C.c_int * 2)(3, 4)
    axes = (C.c_int * 1)(5)
    st = L.ag_reduce_sum_f32(null, null, null, shape, 2, axes, 1, 0, null, 0)
    assert st == 5
    # float-encoded argmax cannot address more than 2^24 elements
    one = C.c_void_p(16)  # never dereferenced: validation fails first
    st = L.ag_maxpool2d_bwd_f32(null, one, one, null, one, 1, 1, 4100, 4100, 2, 0, 2)
    assert st == 4 and b"2^24" in L.ag_last_error()
    # empty problems are accepted without touching the device
    assert L.ag_im2col_f32(null, null, null, 0, 3, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1) == 0
    assert L.ag_gemm_f32(null, 0, 0, 0, 4, 4, 1.0, null, 4, 0, null, 4, 0, 0.0, null, 4, 0, 1) == 0


def test_column_free_geometry_support_is_decided_on_the_host(capi):
    """Which geometries the implicit (column-free) convolution takes is pure host arithmetic."""
    L = capi.lib()
    # the headline (stride 1) and its stride-2 variant at B = 256
    assert L.ag_conv2d_nocols_scratch_floats(256, 64, 56, 56, 128, 3, 3, 1, 1, 1) > 0
    assert L.ag_conv2d_nocols_scratch_floats(256, 64, 56, 56, 128, 3, 3, 1, 2, 1) > 0
    assert L.ag_conv2d_filter_grad_nocols_f32_workspace(256, 64, 56, 56, 128, 3, 3, 1, 2, 1) > 0
    assert L.ag_conv_input_grad_scratch_floats(256, 128, 28, 28, 64, 3, 3, 1, 2, 1, 56, 56) > 0
    assert L.ag_conv_input_grad_scratch_floats(256, 128, 28, 28, 64, 3, 3, 1, 2, 1, 55, 55) > 0   # the reference's reconstructed extent
    # the 4x4 stride-2 transposed convolution of configuration 5 is the input-gradient form
    assert L.ag_conv_input_grad_scratch_floats(32, 128, 14, 14, 64, 4, 4, 1, 2, 1, 28, 28) > 0
    # not taken: dilation, stride 3, channel counts that are not multiples of 32, a gradient of the wrong extent
    assert L.ag_conv2d_nocols_scratch_floats(32, 256, 14, 14, 256, 3, 3, 2, 1, 2) > 0       # 14 x 14 images, 256 filters
    assert L.ag_conv2d_nocols_scratch_floats(64, 128, 28, 28, 128, 3, 3, 2, 1, 2) > 0       # dilated stride 1
    assert L.ag_conv2d_filter_grad_nocols_f32_workspace(64, 128, 28, 28, 128, 3, 3, 2, 1, 2) > 0
    assert L.ag_conv2d_filter_grad_nocols_f32_workspace(64, 128, 28, 28, 128, 3, 3, 1, 1, 2) > 0    # any padding
    assert L.ag_conv2d_nocols_scratch_floats(32, 64, 28, 28, 64, 3, 3, 2, 2, 2) == 0          # dilated stride 2
    assert L.ag_conv2d_nocols_scratch_floats(8, 64, 56, 56, 128, 3, 3, 1, 3, 1) == 0
    assert L.ag_conv2d_nocols_scratch_floats(8, 48, 56, 56, 128, 3, 3, 1, 2, 1) == 0
    assert L.ag_conv_input_grad_scratch_floats(8, 128, 27, 27, 64, 3, 3, 1, 2, 1, 56, 56) == 0
