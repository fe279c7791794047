"""Shared test utilities: seeded inputs and strict bit-level comparison."""
import torch


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def weight_like(rows, cols, seed=0, dtype=torch.float32, std=0.02, outlier_frac=0.001, outlier_mul=20.0):
    """~N(0, std) with a fraction of entries scaled up (outliers), as the baseline configs describe."""
    g = gen(seed)
    w = torch.randn(rows, cols, generator=g) * std
    n = w.numel()
    k = int(outlier_frac * n)
    if k:
        idx = torch.randperm(n, generator=g)[:k]
        w.view(-1)[idx] *= outlier_mul
    return w.to(dtype)


def bits(t: torch.Tensor) -> torch.Tensor:
    """Raw bit pattern as an integer tensor (so -0.0 != +0.0 and NaNs compare)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.view(torch.int32)
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16)
    if t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return t.view(torch.uint8)
    return t


def assert_bit_equal(a, b, what=''):
    assert a.dtype == b.dtype, f'{what}: dtype {a.dtype} vs {b.dtype}'
    assert tuple(a.shape) == tuple(b.shape), f'{what}: shape {tuple(a.shape)} vs {tuple(b.shape)}'
    ba, bb = bits(a), bits(b)
    if not torch.equal(ba, bb):
        bad = (ba != bb)
        n = int(bad.sum())
        i = bad.flatten().nonzero()[0].item()
        raise AssertionError(f'{what}: {n}/{ba.numel()} elements differ; first at flat index {i}: '
                             f'{a.detach().cpu().flatten()[i].item()!r} vs {b.detach().cpu().flatten()[i].item()!r}')
