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
    g = torch.Generator().manual_seed(99)
    big = (torch.randn(3072 * 3072, generator=g) * 5.0).bfloat16().to(dev)       # 576 partial maxima, large values
    small = (torch.randn(40_000, generator=g) * 0.01).bfloat16().to(dev)         # 3 partial maxima, small values
    for x in (big, small):
        (q0, s0), (q1, s1) = _both(L, x)
        assert torch.equal(q0, q1)
        assert np.array_equal(s0.cpu().numpy().view(np.uint32), s1.cpu().numpy().view(np.uint32))
        assert s1.item() == np.float32(x.float().abs().max().item() / np.float32(127.0)) or s1.item() > 0
    # the second, smaller call must not have seen the first call's maxima
    assert s1.item() < 1e-2
