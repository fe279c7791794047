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
    assert lib.lcq_sq_err_mean_static(L.ptr(x), L.ptr(x), L.i32(7), L.i64(64), L.ptr(out), L.stream()) == -3      # no such type code
    with pytest.raises(L.LcqError, match='stated maximum'):
        L.check(-6, 'lcq_sq_err_mean_static')


def test_static_scratch_entry_point_in_a_captured_graph(dev):
    """After one call outside any capture (the first call on a device looks the array's address up, which is not a
    kernel launch), calls are plain kernel launches: two of them captured into one graph, replayed several times with
    eager work and synchronisations in between, give the workspace entry point's result on every replay."""
    from lightcompress_amd import _lib as L
    lib = L.lib()
    n1, n2 = 3 * 1024 * 1024, 48 * 1024
    a1, b1 = (t.to(dev) for t in _pair(n1, torch.bfloat16, 100))
    a2, b2 = (t.to(dev) for t in _pair(n2, torch.float32, 102))
    ws = torch.empty(lib.lcq_awq_workspace_bytes(L.i64(4096)), dtype=torch.uint8, device=dev)
    out1, out2 = torch.zeros(1, device=dev), torch.zeros(1, device=dev)
    want1, want2 = torch.zeros(1, device=dev), torch.zeros(1, device=dev)
    L.check(lib.lcq_sq_err_mean_static(L.ptr(a2), L.ptr(b2), L.i32(L.F32), L.i64(n2), L.ptr(out2), L.stream()), 'warm-up')
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        L.check(lib.lcq_sq_err_mean_static(L.ptr(a1), L.ptr(b1), L.i32(L.BF16), L.i64(n1), L.ptr(out1), L.stream()), 'captured 1')
        L.check(lib.lcq_sq_err_mean_static(L.ptr(a2), L.ptr(b2), L.i32(L.F32), L.i64(n2), L.ptr(out2), L.stream()), 'captured 2')
    for rep in range(4):
        a1.mul_(1.0 + 0.25 * rep)                          # eager work between the replays: new inputs every time
        b2.add_(0.125)
        L.check(lib.lcq_sq_err_mean(L.ptr(a1), L.ptr(b1), L.i32(L.BF16), L.i64(n1), L.ptr(want1), L.ptr(ws), L.stream()), 'eager 1')
        L.check(lib.lcq_sq_err_mean(L.ptr(a2), L.ptr(b2), L.i32(L.F32), L.i64(n2), L.ptr(want2), L.ptr(ws), L.stream()), 'eager 2')
        out1.fill_(-1.0)
        out2.fill_(-1.0)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out1.view(torch.int32), want1.view(torch.int32)), (rep, float(out1), float(want1))
        assert torch.equal(out2.view(torch.int32), want2.view(torch.int32)), (rep, float(out2), float(want2))
