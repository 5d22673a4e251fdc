"""The allocation-free tensorwise quantiser (i8f_quant_tensorwise_static, partial maxima in a device
array of the library) against the workspace variant it mirrors, through the C ABI, bit for bit:
two calls in a row on the same GPU, the second on a smaller tensor, so that stale partial maxima of the
first call would show."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _both(L, x):
    lib = L.lib()
    n = x.numel()
    stream = ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream)
    out = []
    for static in (False, True):
        q = torch.full((n,), 77, dtype=torch.int8, device=x.device)
        s = torch.full((1,), -1.0, dtype=torch.float32, device=x.device)
        if static:
            rc = lib.i8f_quant_tensorwise_static(x.data_ptr(), L.dtype_code(x.dtype), n, q.data_ptr(), s.data_ptr(), stream)
        else:
            ws = torch.empty(1024, dtype=torch.float32, device=x.device)
            rc = lib.i8f_quant_tensorwise(x.data_ptr(), L.dtype_code(x.dtype), n, q.data_ptr(), s.data_ptr(), ws.data_ptr(),
                                          ws.numel() * 4, stream)
        assert rc == 0, rc
        out.append((q, s))
    torch.cuda.synchronize()
    return out


def test_static_scratch_variant_equals_workspace_variant_twice(L, dev):
    import oracle as O

    g = torch.Generator().manual_seed(99)
    big = (torch.randn(3072 * 3072, generator=g) * 5.0).bfloat16()       # 576 partial maxima, large values
    small = (torch.randn(40_000, generator=g) * 0.01).bfloat16()         # 3 partial maxima, small values
    for x_cpu in (big, small):
        x = x_cpu.to(dev)
        (q0, s0), (q1, s1) = _both(L, x)
        assert torch.equal(q0, q1)
        assert np.array_equal(s0.cpu().numpy().view(np.uint32), s1.cpu().numpy().view(np.uint32))
        # ... and both are the oracle's bits (the reference's quantize_int8_tensorwise restated in C)
        xa, code = O.from_torch(x_cpu)
        want_q, want_s = O.quant_tensorwise(xa, code)
        assert np.array_equal(q1.cpu().numpy(), want_q.reshape(-1))
        assert np.array_equal(s1.cpu().numpy().view(np.uint32), np.asarray(want_s, dtype=np.float32).reshape(-1).view(np.uint32))
    # the second, smaller call must not have seen the first call's maxima
    assert s1.item() < 1e-2


def test_static_scratch_variant_allocates_no_device_memory(L, dev):
    """What the entry point is for: after one call that has resolved the address of the library's device array, a
    call changes neither the free memory of the device (hipMemGetInfo) nor anything torch's allocator holds (the
    outputs are allocated beforehand)."""
    lib = L.lib()
    x = (torch.randn(1 << 20, device=dev) * 3.0).bfloat16()
    q = torch.empty(x.numel(), dtype=torch.int8, device=dev)
    s = torch.empty(1, dtype=torch.float32, device=dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    def call():
        rc = lib.i8f_quant_tensorwise_static(x.data_ptr(), L.dtype_code(x.dtype), x.numel(), q.data_ptr(), s.data_ptr(), stream)
        assert rc == 0, rc

    call()                                   # the first call on a device looks the array up
    torch.cuda.synchronize()
    free0, _total = torch.cuda.mem_get_info(dev)
    torch_alloc0, torch_reserved0 = torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev)
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    free1, _total = torch.cuda.mem_get_info(dev)
    assert free1 == free0, f"device free memory changed by {free0 - free1} bytes"
    assert torch.cuda.memory_allocated(dev) == torch_alloc0 and torch.cuda.memory_reserved(dev) == torch_reserved0
    assert s.item() == np.float32(np.float32(x.float().abs().max().item()) / np.float32(127.0))
