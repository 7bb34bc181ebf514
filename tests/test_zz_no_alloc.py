"""The matrix product that allocates nothing (xrt_linear_static), called through ctypes.

Its partial sums go to a fixed array that the library holds on the GPU, so every call shares
it: two calls in a row, the second with a smaller product, must each give what xrt_linear
gives with a workspace of the caller's (the same kernels in the same order: bit for bit), and
what the first call left in the array must not reach the second's result.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

def library():
    from xeno_rt_amd.ops import build
    path = build.find_library() or build.build()
    lib = ctypes.CDLL(path)
    lib.xrt_last_error.restype = ctypes.c_char_p
    lib.xrt_linear_workspace.restype = ctypes.c_long
    lib.xrt_linear.restype = ctypes.c_int
    lib.xrt_linear_static.restype = ctypes.c_int
    lib.xrt_linear_static_floats.restype = ctypes.c_long
    return lib


def pointer(tensor):
    return ctypes.c_void_p(0 if tensor is None else tensor.data_ptr())


def operands(m, n, k, mode, seed):
    generator = torch.Generator(device="cuda").manual_seed(seed)
    rows_w = 2 * n if mode == 2 else n
    a = torch.randn((m, k), generator=generator, device="cuda").to(torch.bfloat16)
    w = (torch.randn((rows_w, k), generator=generator, device="cuda") * 0.05).to(torch.bfloat16)
    start = torch.randn((m, n), generator=generator, device="cuda")       # what an accumulating product adds to
    return a, w, start


def both_ways(lib, m, n, k, mode, seed):
    """(result with the caller's workspace, result with the library's fixed array, floats of partial sums)."""
    a, w, start = operands(m, n, k, mode, seed)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = int(lib.xrt_linear_workspace(pointer(a), pointer(w), 1, m, n, k, mode))
    out_dtype = 0 if mode == 1 else 1
    fresh = lambda: start.clone() if mode == 1 else torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    want, got = fresh(), fresh()
    workspace = torch.empty(max(need, 1), dtype=torch.float32, device="cuda")
    status = lib.xrt_linear(pointer(a), pointer(w), 1, pointer(want), out_dtype, m, n, k, mode,
                            pointer(workspace), ctypes.c_long(need), stream)
    assert status == 0, lib.xrt_last_error().decode()
    status = lib.xrt_linear_static(pointer(a), pointer(w), 1, pointer(got), out_dtype, m, n, k, mode, stream)
    assert status == 0, lib.xrt_last_error().decode()
    torch.cuda.synchronize()
    # and both against a plain product
    plain = a.float() @ w.float().t()
    if mode == 2:
        gate, up = plain[:, :n], plain[:, n:]
        plain = gate / (1.0 + torch.exp(-gate)) * up
    elif mode == 1:
        plain = plain + start
    assert float((want.float() - plain).abs().max()) <= 2e-2 * float(plain.abs().max())
    return want, got, need


def test_two_calls_in_a_row_share_the_fixed_array():
    lib = library()
    # a product whose partial sums fill a good part of the array, then a smaller one of another mode,
    # then one that needs no partial sums at all
    for m, n, k, mode, seed in ((64, 4096, 4096, 1, 1), (24, 1024, 2048, 0, 2), (40, 1536, 1024, 2, 3),
                                (8, 512, 256, 0, 4)):
        want, got, need = both_ways(lib, m, n, k, mode, seed)
        assert need <= int(lib.xrt_linear_static_floats())
        if m > 16 and mode != 2:
            assert need > 0, "this product was meant to be split along k"
        assert torch.equal(want, got), (m, n, k, mode)


def test_a_product_beyond_the_fixed_array_is_refused_and_nothing_is_written():
    lib = library()
    m, n, k = 1024, 2048, 8192              # large tiles that split k in eight: 16 Mi floats of partial sums
    a, w, _ = operands(m, n, k, 0, 5)
    need = int(lib.xrt_linear_workspace(pointer(a), pointer(w), 1, m, n, k, 0))
    assert need > int(lib.xrt_linear_static_floats())
    out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    status = lib.xrt_linear_static(pointer(a), pointer(w), 1, pointer(out), 1, m, n, k, 0, stream)
    assert status != 0
    message = lib.xrt_last_error().decode()
    assert "fixed buffer" in message and str(need) in message
    torch.cuda.synchronize()
    assert bool((out == 7.0).all())


def test_the_calls_allocate_no_device_memory():
    """What the entry point is for: after a first call (which may load the code object and asks for the array's
    address), calls of every kind, split along k or not, leave the device's free memory as it was."""
    lib = library()
    cases = [(operands(m, n, k, mode, seed), (m, n, k, mode))
             for m, n, k, mode, seed in ((64, 4096, 4096, 1, 1), (24, 1024, 2048, 0, 2), (40, 1536, 1024, 2, 3), (8, 512, 256, 0, 4))]
    outs = [start.clone() if mode == 1 else torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
            for (_, _, start), (m, n, k, mode) in cases]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call_all():
        for ((a, w, _), (m, n, k, mode)), out in zip(cases, outs):
            status = lib.xrt_linear_static(pointer(a), pointer(w), 1, pointer(out), 0 if mode == 1 else 1, m, n, k, mode, stream)
            assert status == 0, lib.xrt_last_error().decode()

    call_all()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        call_all()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"free device memory went from {free_before} to {free_after} bytes"
