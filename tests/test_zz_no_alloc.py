"""The product entry point that allocates nothing (vt_linear_bf16_noalloc), called through ctypes as a caller
without torch's allocator would: its partial sums go into an array that the library's code object brings, so the
caller passes inputs and outputs only.  Checked against the entry point it is a variant of (vt_linear_bf16 with
a workspace) on two calls in a row, the second with a smaller input, which finds the first call's partial sums
still lying in the array."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _lib(half):
    from vt_transformer_amd.kernels.build import load_lib
    lib = load_lib("vt_gemm_bf16", half=half)
    lib.vt_linear_bf16_workspace.restype = ctypes.c_longlong
    lib.vt_last_error.restype = ctypes.c_char_p
    return lib


@pytest.mark.parametrize("lp", [torch.bfloat16, torch.float16])
def test_noalloc_product_equals_the_product_with_a_workspace_twice_in_a_row(lp):
    """Both 16-bit builds of the library carry an array and a per-device pointer of their own."""
    from vt_transformer_amd.kernels import ops
    lib = _lib(lp == torch.float16)
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    gen = torch.Generator(device="cpu").manual_seed(5)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # shapes whose k range is split over blocks (few rows of W, a long k), first 48 rows, then 40 of a smaller W;
    # then one that needs no scratch memory at all (8 rows: the array is not even looked up)
    for n, m, k in ((48, 3584, 18944), (40, 1536, 8960), (8, 1536, 8960)):
        need = int(lib.vt_linear_bf16_workspace(n, m, k, 0))
        assert (need > 0) == (n > 16), "the first two shapes use scratch memory, the third does not"
        x = (torch.randn(n, k, generator=gen) * 0.5).to(lp).to(dev)
        w = (torch.randn(m, k, generator=gen) * 0.02).to(lp).to(dev)
        bias = torch.randn(m, generator=gen).to(dev)
        packed = ops.pack_matrix_bf16(w)
        want = torch.empty(n, m, dtype=torch.float32, device=dev)
        work = torch.empty(max(need, 1), dtype=torch.float32, device=dev)
        rc = lib.vt_linear_bf16(_ptr(x), _ptr(packed.data), _ptr(bias), _ptr(want), 0, _ptr(work if need else None),
                                n, m, k, stream)
        assert rc == 0, lib.vt_last_error().decode()
        got = torch.full((n, m), float("nan"), dtype=torch.float32, device=dev)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(dev)
        rc = lib.vt_linear_bf16_noalloc(_ptr(x), _ptr(packed.data), _ptr(bias), _ptr(got), 0, n, m, k, stream)
        assert rc == 0, lib.vt_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(dev) == before
        assert torch.equal(got, want), (n, m, k)
        # and the product is the product: against float64 on the same 16-bit values
        ref = x.double() @ w.double().t() + bias.double()
        assert float((got.double() - ref).abs().max() / ref.abs().max()) < 1e-5


def test_noalloc_product_refuses_what_its_array_cannot_hold():
    lib = _lib(False)
    n, m, k = 256, 3584, 18944
    assert int(lib.vt_linear_bf16_workspace(n, m, k, 0)) > 4 * 1024 * 1024
    # refused on the host before anything is read: the pointers are never used
    rc = lib.vt_linear_bf16_noalloc(None, None, None, None, 0, n, m, k, None)
    assert rc != 0 and b"built-in" in lib.vt_last_error()
