"""Reduction blocks are per stream: they return to the pool when a stream is destroyed through the library, are
cleared when bound to the next stream, and can be cleared on request."""
import ctypes

import numpy as np
import pytest

from helpers import rng

pytestmark = pytest.mark.gpu


def test_amax_on_more_streams_than_reduction_blocks(pkg, orc):
    """300 create / amax / destroy rounds: the pool holds 256 blocks, so this only works if destroyed streams give
    theirs back (the executor creates and destroys streams per session)."""
    import torch
    L = pkg.lib()
    x_np = rng(5).standard_normal(70001, dtype=np.float32)
    x = torch.from_numpy(x_np).cuda()
    ref = orc.amax(x_np, orc.F32)
    out = torch.zeros(2, device="cuda")
    for i in range(300):
        s = L.mtrt_cuda_stream_create()
        assert s
        out.fill_(-1.0)
        torch.cuda.synchronize()
        pkg.check(L.mtrt_hip_amax(s, x.data_ptr(), pkg.F32, x.numel(), 127.0, out.data_ptr(), out.data_ptr() + 4))
        L.mtrt_cuda_stream_sync(s)
        assert np.float32(out[0].item()).tobytes() == ref.tobytes(), i
        L.mtrt_cuda_stream_destroy(s)
    # the interpreter flavour of stream destroy gives blocks back as well
    for i in range(300):
        h = ctypes.c_size_t(0)
        assert L.mtrt_lua_cuda_stream_create(ctypes.byref(h)) == 0
        pkg.check(L.mtrt_hip_amax(h.value, x.data_ptr(), pkg.F32, x.numel(), 127.0, out.data_ptr(), out.data_ptr() + 4))
        assert L.mtrt_lua_cuda_stream_destroy(h.value) == 0
    torch.cuda.synchronize()
    assert np.float32(out[0].item()).tobytes() == ref.tobytes()


def test_reset_reductions_keeps_results(pkg, orc):
    import torch
    L = pkg.lib()
    x_np = rng(6).standard_normal(123457, dtype=np.float32)
    x = torch.from_numpy(x_np).cuda()
    s = torch.cuda.current_stream().cuda_stream
    pkg.check(L.mtrt_hip_reset_reductions(s))          # nothing bound yet or already zero: both fine
    a0, _ = pkg.amax(x, 127.0)
    pkg.check(L.mtrt_hip_reset_reductions(s))
    a1, _ = pkg.amax(x, 127.0)
    torch.cuda.synchronize()
    ref = orc.amax(x_np, orc.F32)
    assert np.float32(a0.item()).tobytes() == ref.tobytes() == np.float32(a1.item()).tobytes()
