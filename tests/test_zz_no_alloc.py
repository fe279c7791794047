"""lcq_sq_err_mean_static: the squared-error entry point that allocates nothing (its partial sums live in an array
inside the library's device image) must give lcq_sq_err_mean's result bit for bit, call after call."""
import pytest
import torch

from tests.helpers import gen

pytestmark = pytest.mark.gpu


def _pair(n, dtype, seed):
    a = torch.randn(n, generator=gen(seed)).to(dtype)
    b = (a.float() + 0.1 * torch.randn(n, generator=gen(seed + 1))).to(dtype)
    return a, b


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
def test_static_scratch_entry_point_matches_the_workspace_one(dev, dtype):
    from lightcompress_amd import _lib as L
    lib = L.lib()
    ws = torch.empty(lib.lcq_awq_workspace_bytes(L.i64(4096)), dtype=torch.uint8, device=dev)
    code = L.i32(L.dtype_code(dtype))
    # two calls in a row, the second on a smaller input (it must not see the first call's partial sums), then a
    # larger one again and a tiny one
    for i, n in enumerate([8192 * 256 * 8 * 3 + 4096, 40 * 1024, 5 * 1024 * 1024, 64]):
        a, b = _pair(n, dtype, 10 * i)
        ad, bd = a.to(dev), b.to(dev)
        want = torch.zeros(1, device=dev)
        got = torch.full((1,), -1.0, device=dev)
        L.check(lib.lcq_sq_err_mean(L.ptr(ad), L.ptr(bd), code, L.i64(n), L.ptr(want), L.ptr(ws), L.stream()), 'workspace')
        L.check(lib.lcq_sq_err_mean_static(L.ptr(ad), L.ptr(bd), code, L.i64(n), L.ptr(got), L.stream()), 'static')
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (n, float(got), float(want))
        ref = float((a - b).float().pow(2).mean())
        assert abs(float(got) - ref) <= 1e-5 * ref


def test_static_scratch_entry_point_rejects_what_it_cannot_hold(dev):
    from lightcompress_amd import _lib as L
    lib = L.lib()
    x = torch.zeros(64, device=dev)
    out = torch.zeros(1, device=dev)
    too_big = (1 << 34) + 8
    assert lib.lcq_sq_err_mean_static(L.ptr(x), L.ptr(x), L.i32(L.F32), L.i64(too_big), L.ptr(out), L.stream()) == -6
    assert lib.lcq_sq_err_mean_static(L.ptr(x), L.ptr(x), L.i32(L.F32), L.i64(0), L.ptr(out), L.stream()) == -1
    assert lib.lcq_sq_err_mean_static(L.ptr(x), L.ptr(x), L.i32(L.F16), L.i64(64), L.ptr(out), L.stream()) == -3
    with pytest.raises(L.LcqError, match='stated maximum'):
        L.check(-6, 'lcq_sq_err_mean_static')
