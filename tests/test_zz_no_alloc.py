"""The entry point that allocates nothing (ag_matmul_f32_noalloc): through the C ABI, against
ag_matmul_f32 with a caller workspace -- same kernels, same slices, so the results must be
bit-identical -- on two calls in a row, the second with a smaller input, and against the f64
product.  torch.cuda.memory_allocated() must not move across the calls."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    from rust_autograd_amd import capi, kernels
    assert torch.cuda.is_available()
    return torch, capi, kernels


def _both(torch, capi, K, a, b, ta, tb):
    """(ag_matmul_f32 result, ag_matmul_f32_noalloc result) for op(a) . op(b)."""
    L = capi.lib()
    m, k = (a.shape[1], a.shape[0]) if ta else a.shape
    n = b.shape[0] if tb else b.shape[1]
    ref = K.matmul(a, b, ta, tb)
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=a.device)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    def call():
        capi.check(L.ag_matmul_f32_noalloc(stream, int(ta), int(tb), m, n, k, C.c_void_p(a.data_ptr()), a.shape[1],
                                           C.c_void_p(b.data_ptr()), b.shape[1], C.c_void_p(out.data_ptr()), n))

    # A first call may load the kernel's code object and look the array's address up; from then on nothing may
    # change the device's free memory: torch's counter only sees torch's own allocator, hipMemGetInfo (what
    # mem_get_info reads) sees a hipMalloc or hipFree from anywhere in the process.
    call()
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    out.fill_(float("nan"))
    call()
    torch.cuda.synchronize()
    call()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory moved during a call that must not allocate"
    return ref, out


def test_no_alloc_matmul_matches_workspace_matmul_twice_then_smaller(env):
    torch, capi, K = env
    L = capi.lib()
    rng = np.random.default_rng(99)
    dev = torch.device("cuda:0")
    # the dense layer of the small CNN ([128,3136].[3136,10], sliced contraction), then a smaller
    # sliced product, then a transposed one, then one that is not sliced at all
    cases = [((128, 3136), (3136, 10), False, False),
             ((64, 1024), (1024, 24), False, False),
             ((2048, 48), (2048, 40), True, False),
             ((96, 80), (80, 72), False, False)]
    sliced = 0
    for sa, sb, ta, tb in cases:
        a_h = rng.standard_normal(sa).astype(np.float32)
        b_h = rng.standard_normal(sb).astype(np.float32)
        a, b = torch.from_numpy(a_h).to(dev), torch.from_numpy(b_h).to(dev)
        m, k = (sa[1], sa[0]) if ta else sa
        n = sb[0] if tb else sb[1]
        sliced += L.ag_matmul_f32_workspace(m, n, k) > 16
        ref, out = _both(torch, capi, K, a, b, ta, tb)
        assert torch.equal(ref, out), f"case {sa}x{sb}: differs from ag_matmul_f32"
        truth = (a_h.T if ta else a_h).astype(np.float64) @ (b_h.T if tb else b_h).astype(np.float64)
        absdot = np.abs(a_h.T if ta else a_h).astype(np.float64) @ np.abs(b_h.T if tb else b_h).astype(np.float64)
        assert (np.abs(out.cpu().numpy() - truth) / absdot).max() <= 2e-6
    assert sliced >= 3, "the cases no longer exercise the scratch array"


def test_no_alloc_matmul_integer_exact_and_repeatable(env):
    torch, capi, K = env
    rng = np.random.default_rng(5)
    dev = torch.device("cuda:0")
    a_h = rng.integers(-4, 5, (64, 4096)).astype(np.float32)
    b_h = rng.integers(-4, 5, (4096, 16)).astype(np.float32)
    a, b = torch.from_numpy(a_h).to(dev), torch.from_numpy(b_h).to(dev)
    want = (a_h.astype(np.int64) @ b_h.astype(np.int64)).astype(np.float32)
    for _ in range(2):  # the second call meets the first call's partial sums in the array
        _, out = _both(torch, capi, K, a, b, False, False)
        assert np.array_equal(out.cpu().numpy(), want)


def test_no_alloc_matmul_refuses_what_exceeds_the_fixed_array(env):
    torch, capi, K = env
    L = capi.lib()
    cap = L.ag_matmul_f32_static_scratch_bytes()
    assert cap == 4 << 20
    # few output tiles but a very long contraction: the slices' partial sums exceed 4 MiB
    m, n, k = 448, 504, 20480
    need = L.ag_matmul_f32_workspace(m, n, k)
    assert need > cap
    one = C.c_void_p(256)  # never dereferenced: refused on the host
    st = L.ag_matmul_f32_noalloc(C.c_void_p(0), 0, 0, m, n, k, one, k, one, n, one, n)
    assert st == 4 and b"fixed array" in L.ag_last_error()
