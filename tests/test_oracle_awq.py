"""Pins the AWQ oracle without a GPU: ratio 0 is plain RTN, the scale
normalisation, and a brute-force fp64 grid search on a tiny SwiGLU MLP."""
import torch

from oracle import awq_ref as A, quant_ref as Q
from tests.helpers import gen


def swiglu(x, w):
    h = torch.nn.functional.silu(x @ w['gate'].t()) * (x @ w['up'].t())
    return h @ w['down'].t() if 'down' in w else h


def tiny_case(dtype, seed=0, T=64, K=256, I=384):
    g = gen(seed)
    sigma = torch.exp(torch.randn(K, generator=g))
    x = (torch.randn(2, T, K, generator=g) * sigma).to(dtype)
    w = {'gate': (torch.randn(I, K, generator=g) * 0.02).to(dtype), 'up': (torch.randn(I, K, generator=g) * 0.02).to(dtype)}
    down = (torch.randn(K, I, generator=g) * 0.02).to(dtype)
    return x, w, down


def test_ratio_zero_is_plain_rtn_and_scales_are_normalised():
    x, w, down = tiny_case(torch.float32)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    s0 = A.get_scales(x, None, 0.0)
    assert torch.equal(s0, torch.ones_like(s0))
    assert torch.equal(A.scale_and_fake_quant(w['gate'], s0, spec), Q.int_fake_quant_dynamic(spec, w['gate']))
    assert torch.equal(A.scaling_input(x, s0), x)
    for r in (0.25, 0.5, 0.95):
        s = A.get_scales(x, None, r)
        assert abs(float(s.max() * s.min()) - 1.0) < 1e-5
        # scales follow the activation magnitude: the ordering of channels is that of mean|x|
        assert torch.equal(torch.argsort(s), torch.argsort(A.act_scale(x).pow(r).clamp(min=1e-4)))
    # closed form of the activation statistic
    assert torch.allclose(A.act_scale(x), x.abs().reshape(-1, 256).sum(0) / 128, rtol=1e-6)


def test_weight_scale_closed_form():
    _, w, _ = tiny_case(torch.float32, seed=1)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    ws = A.weight_scale([w['gate'], w['up']], spec)
    ref = 0
    for m in (w['gate'], w['up']):
        a = m.abs().reshape(m.shape[0], -1, 128)
        ref = ref + (a / a.amax(-1, keepdim=True)).reshape(m.shape).mean(0)
    assert torch.allclose(ws, ref / 2, rtol=1e-6)
    assert float(ws.max()) <= 1.0


def test_grid_search_matches_bruteforce_fp64():
    x, w, down = tiny_case(torch.float64, seed=2)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: swiglu(xx, dict(ww, down=down))
    best, losses = A.search_scale(w, x, fwd, spec)
    assert len(losses) == 20
    # independent evaluation of every grid point
    org = fwd(x, w)
    xm = x.abs().reshape(-1, x.shape[-1]).mean(0)
    brute = []
    for n in range(20):
        s = xm.pow(n / 20).clamp(min=1e-4)
        s = s / (s.max() * s.min()).sqrt()
        wq = {k: Q.int_fake_quant_dynamic(spec, v * s) for k, v in w.items()}
        brute.append(float(((org - fwd(x / s, wq)) ** 2).mean()))
    assert torch.allclose(torch.tensor(losses), torch.tensor(brute), rtol=1e-9)
    k = min(range(20), key=lambda i: brute[i])
    s = xm.pow(k / 20).clamp(min=1e-4)
    assert torch.allclose(best, s / (s.max() * s.min()).sqrt())
    # activation-aware scaling beats plain RTN on outlier channels
    assert min(brute) < brute[0]
