"""The entry point of the kernel library that allocates nothing (``pta_gemm_splitk_bf16_static``), called
through ctypes as a caller without an allocator would, against the entry point that takes a workspace."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _both_ways(lib, M, N, K, seed, with_tail_terms):
    """The product through the workspace entry point and through the one that allocates nothing."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn((M, K), generator=g, device="cuda").to(torch.bfloat16)
    w = (torch.randn((N, K), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
    bias = torch.randn((N,), generator=g, device="cuda") if with_tail_terms else None
    add1 = torch.randn((M, N), generator=g, device="cuda").to(torch.bfloat16) if with_tail_terms else None
    act = 1 if with_tail_terms else 0  # the exact GELU, or none
    parts = lib.pta_gemm_splitk_parts(N, K, 0, 0)
    part = torch.empty((parts, M, N), dtype=torch.float32, device="cuda")
    want = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.pta_gemm_splitk_bf16(_ptr(want), _ptr(part), _ptr(x), _ptr(w), _ptr(bias), _ptr(add1), None, M, N, K, act, 0,
                                  0, 0, 0, 0, 1, stream)
    assert rc == 0, lib.pta_last_error().decode()
    # once to warm up (the first call on a device looks the array's address up, and the code object is loaded), then
    # the call whose memory is watched: torch's own counter, and the driver's count of free device memory, which
    # also sees an allocation that does not go through torch
    rc = lib.pta_gemm_splitk_bf16_static(_ptr(got), _ptr(x), _ptr(w), _ptr(bias), _ptr(add1), None, M, N, K, act, 0, stream)
    assert rc == 0, lib.pta_last_error().decode()
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    rc = lib.pta_gemm_splitk_bf16_static(_ptr(got), _ptr(x), _ptr(w), _ptr(bias), _ptr(add1), None, M, N, K, act, 0, stream)
    assert rc == 0, lib.pta_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
    ref = x.float() @ w.float().t()
    return got, want, ref, parts


def test_the_entry_point_that_allocates_nothing_equals_the_one_with_a_workspace():
    from pytorch_transformers_amd import ops

    lib = ops.load_library()
    lib.pta_gemm_splitk_static_floats.restype = ctypes.c_long
    limit = lib.pta_gemm_splitk_static_floats()
    assert limit == 4 * 1024 * 1024
    # two calls in a row on the same GPU share the library's array: the second, smaller one must not see the
    # first one's partial sums
    for (M, N, K), tail_terms, seed in (((96, 1184, 4672), True, 1), ((24, 328, 1096), False, 2)):
        got, want, ref, parts = _both_ways(lib, M, N, K, seed, tail_terms)
        assert parts > 1, "the shape must be one that is split over K, or the workspace is not used"
        assert parts * M * N <= limit
        assert torch.equal(got, want), f"M={M} N={N} K={K}: differs from the workspace entry point"
        if not tail_terms:
            err = float((got.float() - ref).abs().max() / ref.abs().max())
            assert err < 2e-2, f"M={M} N={N} K={K}: off the 32-bit product by {err:.3e} of its scale"


def test_it_refuses_a_product_beyond_its_workspace():
    from pytorch_transformers_amd import ops

    lib = ops.load_library()
    lib.pta_last_error.restype = ctypes.c_char_p
    M, N, K = 256, 8192, 8192  # ranges x 256 x 8192 partial sums are more than the array holds
    assert lib.pta_gemm_splitk_parts(N, K, 0, 0) * M * N > 4 * 1024 * 1024
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((N, K), dtype=torch.bfloat16, device="cuda")
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    rc = lib.pta_gemm_splitk_bf16_static(_ptr(y), _ptr(x), _ptr(w), None, None, None, M, N, K, 0, 0,
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc != 0
    assert "workspace holds" in lib.pta_last_error().decode()
