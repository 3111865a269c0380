"""The entry point that allocates nothing, nb_bmv_bn_act_static_i64 (workspace in the library's fixed device array),
called through the C ABI and compared bit for bit with nb_bmv_bn_act_i64 (caller-supplied workspace): two calls in a
row, the second with a smaller input, so that what the first call left in the shared array must not leak into the
second; bool and packed output; the size limit is rejected with a clear error and nothing launched."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(lib, g, Z, M, Kw, pack):
    K = 64 * Kw - 3
    A = torch.from_numpy(g.integers(-2 ** 63, 2 ** 63, size=(Z, M, Kw), dtype=np.int64)).cuda()
    x = torch.from_numpy(g.integers(-2 ** 63, 2 ** 63, size=(Z, Kw), dtype=np.int64)).cuda()
    bias = torch.from_numpy((g.standard_normal(M) * 4).astype(np.float16)).cuda()
    noise = torch.from_numpy(((g.random((Z, M)) - 0.5) * 6).astype(np.float16)).cuda()
    shape, dt = ((Z, (M + 63) // 64), torch.int64) if pack else ((Z, M), torch.bool)
    need = lib.nb_bmv_bn_workspace_bytes(Z, M)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = torch.empty(shape, dtype=dt, device="cuda")
    got = torch.empty(shape, dtype=dt, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    args = (A.data_ptr(), x.data_ptr(), bias.data_ptr(), noise.data_ptr(), Z, M, Kw, K, 1 if pack else 0)
    assert lib.nb_bmv_bn_act_i64(want.data_ptr(), *args, ws.data_ptr(), need, st) == 0, lib.nb_last_error_string()
    assert lib.nb_bmv_bn_act_static_i64(got.data_ptr(), *args, st) == 0, lib.nb_last_error_string()
    torch.cuda.synchronize()
    assert torch.equal(got, want), "Z=%d M=%d Kw=%d pack=%d" % (Z, M, Kw, pack)
    assert bool(want.any()) and not bool(want.all()) if not pack else True


def test_static_workspace_entry_point_equals_the_workspace_one():
    assert torch.cuda.is_available()
    from nesgpu_amd import _lib
    lib = _lib.load()
    assert lib.nb_bmv_bn_static_bytes() == (4 << 20) + (64 << 10)
    g = np.random.default_rng(2024)
    for pack in (False, True):
        _case(lib, g, 512, 1024, 16, pack)        # fills half of the fixed array
        _case(lib, g, 37, 130, 5, pack)           # a smaller input straight after it
        _case(lib, g, 1024, 1024, 4, pack)        # the largest shape that fits: 4 MiB of sums + 8 KiB of totals
    # beyond the fixed array: rejected, nothing launched (dummy pointers are never dereferenced)
    one = ctypes.c_void_p(256)
    assert lib.nb_bmv_bn_act_static_i64(one, one, one, one, one, 1100, 1024, 4, 256, 0, None) == 2
    msg = lib.nb_last_error_string()
    assert b"fixed array" in msg and b"bytes" in msg
    assert lib.nb_bmv_bn_act_static_i64(None, None, None, None, None, 0, 1024, 4, 256, 0, None) == 0   # empty
