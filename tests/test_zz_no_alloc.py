"""``oa_grad_norm_bf16_static``: the gradient-norm entry point that allocates
nothing (its partial sums live in a device array inside the library), called
through the C ABI and compared bit for bit with ``oa_grad_norm_bf16``, which
takes the same partial sums through a caller-provided workspace.

Collected last on purpose (file name): a failure here must not hide the other
GPU tests from a run with ``-x``.
"""

from ctypes import c_int64, c_void_p

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16


def _both(lib, grad, ws):
    """(norm bits, sum-of-squares bits) from the workspace entry point and from
    the static-scratch one, on the current stream."""
    n = grad.numel()
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for static in (False, True):
        norm = torch.full((1,), -1.0, dtype=BF16, device="cuda")
        sumsq = torch.full((1,), -1.0, dtype=torch.float32, device="cuda")
        if static:
            rc = lib.oa_grad_norm_bf16_static(c_void_p(grad.data_ptr()), c_int64(n),
                                              c_void_p(norm.data_ptr()),
                                              c_void_p(sumsq.data_ptr()), stream)
        else:
            rc = lib.oa_grad_norm_bf16(c_void_p(grad.data_ptr()), c_int64(n),
                                       c_void_p(norm.data_ptr()), c_void_p(sumsq.data_ptr()),
                                       c_void_p(ws.data_ptr()), stream)
        assert rc == 0, (static, rc)
        torch.cuda.synchronize()
        out.append((int(norm.view(torch.int16).cpu().numpy().view(np.uint16)[0]),
                    int(sumsq.cpu().numpy().view(np.uint32)[0])))
    return out


def test_static_scratch_norm_matches_workspace_norm(oracle):
    from offload_adam_amd import _lib

    lib = _lib.load()
    ws = torch.empty(lib.oa_norm_workspace_bytes(), dtype=torch.uint8, device="cuda")
    gen = torch.Generator().manual_seed(11)
    # two calls in a row, the second smaller: fewer blocks than the first, so the
    # array still holds the first call's partials beyond the second call's
    big = (torch.randn(40_000_003, generator=gen) * 5e-3).to(BF16).cuda()
    small = (torch.randn(70_001, generator=gen) * 5e-3).to(BF16).cuda()
    before = torch.cuda.memory_allocated()
    for grad in (big, small, big[3:1_000_000], small[:1], small[:0]):
        want, got = _both(lib, grad, ws)
        assert got == want, (grad.numel(), want, got)
        host = grad.view(torch.int16).cpu().numpy().view(np.uint16)
        assert abs(got[0] - int(oracle.grad_norm_bf16(host))) <= 1  # 1 bf16 ulp: order of the sum
    assert torch.cuda.memory_allocated() == before


def test_static_scratch_norm_takes_no_memory_from_the_driver():
    """torch's allocator statistics cannot see a hipMalloc inside the library; the
    driver's own count of free device memory can.  Batches of calls (after a first one,
    which looks the array's address up) must leave it where it was."""
    from offload_adam_amd import _lib

    lib = _lib.load()
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    grads = [(torch.randn(n, generator=torch.Generator().manual_seed(n)) * 5e-3).to(BF16).cuda()
             for n in (5_000_011, 300_001, 17)]
    norm = torch.zeros(1, dtype=BF16, device="cuda")
    sumsq = torch.zeros(1, dtype=torch.float32, device="cuda")

    def call(g):
        rc = lib.oa_grad_norm_bf16_static(c_void_p(g.data_ptr()), c_int64(g.numel()),
                                          c_void_p(norm.data_ptr()), c_void_p(sumsq.data_ptr()),
                                          stream)
        assert rc == 0

    for g in grads:
        call(g)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before = torch.cuda.memory_reserved()
    for _ in range(50):
        for g in grads:
            call(g)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_reserved() == reserved_before  # torch itself took nothing either
    assert free_after == free_before, (free_before, free_after)


def test_static_scratch_norm_rejects_sizes_beyond_its_maximum():
    from offload_adam_amd import _lib

    lib = _lib.load()
    g = torch.zeros(16, dtype=BF16, device="cuda")
    norm = torch.full((1,), 7.0, dtype=BF16, device="cuda")
    rc = lib.oa_grad_norm_bf16_static(c_void_p(g.data_ptr()), c_int64((1 << 31) + 1),
                                      c_void_p(norm.data_ptr()), None, None)
    assert rc == -3  # OA_ERANGE, nothing launched
    torch.cuda.synchronize()
    assert norm.item() == 7.0
    assert "beyond" in _lib.error_string(rc)
