"""Seeded random configurations of the quantizers, of GPTQ and of the AWQ search against the oracle.

The other GPU tests pick their configurations by hand; these draw them - type of the tensor and of the qparams, shape
(ragged, single row, single column, fewer columns than a group), bit width, granularity, data (outliers, constant, zero,
tiny, huge, all negative, infinite), rounding options - from a seeded generator, so the cases are the same on every run
and a failure names the draw that caused it.  The bars are those of the hand-picked tests: bit for bit for the
quantizers, summed loss within 1 % for GPTQ, the same grid point and the same scale bits for the AWQ search.
"""
import random
import types

import pytest
import torch

from oracle import awq_ref as A
from oracle import gptq_ref as G
from oracle import quant_ref as Q

pytestmark = pytest.mark.gpu

_VIEW = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}


def _bits(t):
    t = t.cpu().contiguous()
    return t.view(_VIEW[t.element_size()])


def _same(a, b):
    return a.shape == b.shape and a.dtype == b.dtype and torch.equal(_bits(a), _bits(b))


def _differing(a, b):
    if a.shape != b.shape or a.dtype != b.dtype:
        return f'{a.dtype}{tuple(a.shape)} against {b.dtype}{tuple(b.shape)}'
    return f'{int((_bits(a) != _bits(b)).sum())} of {a.numel()} entries differ'


@pytest.fixture(scope='module')
def dev():
    from lightcompress_amd import _lib
    _lib.lib()
    return torch.device('cuda:0')


@pytest.mark.parametrize('seed', [0, 1, 2, 3])
def test_random_integer_quantizer_configs(dev, seed):
    """IntegerQuantizer fake_quant_{weight,act}_dynamic and real_quant_weight_dynamic (quant.py:698-1032)."""
    from lightcompress_amd import IntegerQuantizer
    rng = random.Random(1000 + seed)
    problems = []
    for it in range(60):
        dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        gran = rng.choice(['per_group', 'per_group', 'per_channel', 'per_tensor', 'per_token'])
        bit = rng.choice([2, 3, 4, 4, 5, 6, 8])
        sym = rng.random() < 0.5
        g = rng.choice([16, 32, 64, 128, 256])
        rows = rng.choice([1, 2, 3, 7, 16, 33, 64, 129, 256, 1000])
        if gran == 'per_group':
            cols = g * rng.choice([1, 2, 3, 5, 8, 17, 32])
        else:
            cols = rng.choice([1, 2, 5, 8, 24, 100, 127, 128, 1000, 1001, 4096, 5000, 11008])
        kind = rng.choice(['normal', 'normal', 'outlier', 'const', 'zero', 'tiny', 'huge', 'neg', 'inf'])
        gg = torch.Generator().manual_seed(rng.randrange(1 << 30))
        x = torch.randn(rows, cols, generator=gg)
        if kind == 'outlier':
            x[torch.rand(rows, cols, generator=gg) < 0.01] *= 50
        elif kind == 'const':
            x[:] = 0.37
        elif kind == 'zero':
            x[:] = 0
        elif kind == 'tiny':
            x *= 1e-7
        elif kind == 'huge':
            x *= 1e3 if dtype == torch.float16 else 1e30
        elif kind == 'neg':
            x = -x.abs() - 1
        elif kind == 'inf':
            x[0, 0] = float('inf')
        x = x.to(dtype)
        round_zp = rng.random() < 0.85
        kw = dict(group_size=g) if gran == 'per_group' else {}
        desc = f'draw {it}: {dtype} {gran} w{bit} sym={sym} g={g} ({rows},{cols}) {kind} round_zp={round_zp}'
        spec = Q.IntSpec(bit, sym, gran, group_size=kw.get('group_size', 0), round_zp=round_zp)
        q = IntegerQuantizer(bit, sym, gran, round_zp=round_zp, **kw)
        xd = x.to(dev)
        got = q.fake_quant_act_dynamic(xd) if gran == 'per_token' else q.fake_quant_weight_dynamic(xd)
        want = Q.int_fake_quant_dynamic(spec, x)
        if kind == 'inf':                                  # NaN where torch has NaN, the same bits elsewhere
            g_, w_ = got.cpu(), want
            ok = g_.shape == w_.shape and g_.dtype == w_.dtype and torch.equal(torch.isnan(g_), torch.isnan(w_)) \
                and torch.equal(torch.nan_to_num(g_.float(), 0, 0, 0), torch.nan_to_num(w_.float(), 0, 0, 0))
        else:
            ok = _same(got, want)
        if not ok:
            problems.append(f'{desc}: fake quant, {_differing(got, want)}')
        if round_zp and gran != 'per_token' and kind != 'inf':
            c, s, z = q.real_quant_weight_dynamic(xd)
            oc, os_, oz = Q.int_real_quant_dynamic(spec, x)
            if not (_same(c, oc) and _same(s, os_) and ((z is None and oz is None) or _same(z, oz))):
                problems.append(f'{desc}: real quant')
    assert not problems, '\n'.join(problems)


@pytest.mark.parametrize('seed', [0, 1])
def test_random_float_quantizer_configs(dev, seed):
    """FloatQuantizer with the qtorch rounding model (quant.py:1042-1237)."""
    from lightcompress_amd import FloatQuantizer
    rng = random.Random(2000 + seed)
    problems = []
    for it in range(60):
        dtype = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        gran = rng.choice(['per_channel', 'per_token', 'per_tensor', 'per_group'])
        fmt = rng.choice(['e4m3', 'e5m2', 'e4m3', 'e2m1', 'e3m2'])
        tie = rng.choice(['away', 'even'])
        rows = rng.choice([1, 3, 16, 65, 300])
        g = rng.choice([32, 128])
        cols = g * rng.choice([1, 3, 8]) if gran == 'per_group' else rng.choice([8, 24, 100, 128, 1000, 1001, 7168])
        gg = torch.Generator().manual_seed(rng.randrange(1 << 30))
        x = (torch.randn(rows, cols, generator=gg) * rng.choice([1e-4, 1.0, 300.0])).to(dtype)
        kw = dict(group_size=g) if gran == 'per_group' else {}
        desc = f'draw {it}: {dtype} {gran} {fmt} tie={tie} ({rows},{cols})'
        q = FloatQuantizer(fmt, True, gran, use_qtorch=True, fp_tie=tie, **kw)
        spec = Q.FloatSpec(fmt, gran, group_size=kw.get('group_size', 0), tie=tie)
        xd = x.to(dev)
        got = q.fake_quant_act_dynamic(xd) if gran == 'per_token' else q.fake_quant_weight_dynamic(xd)
        want = Q.float_fake_quant_dynamic(spec, x)
        if not _same(got, want):
            problems.append(f'{desc}: {_differing(got, want)}')
    assert not problems, '\n'.join(problems)


@pytest.mark.parametrize('seed', [0, 1])
def test_random_static_configs(dev, seed):
    """fake_quant_{weight,act}_static and real_quant_weight_static with qparams of the tensor's type or fp32, taken from
    another tensor, with and without an output scale factor (quant.py:1009-1032, 806-838)."""
    from lightcompress_amd import IntegerQuantizer
    rng = random.Random(3000 + seed)
    problems = []
    for it in range(80):
        dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
        qp_dtype = rng.choice([dtype, dtype, torch.float32])
        gran = rng.choice(['per_group', 'per_channel', 'per_tensor', 'per_token'])
        bit = rng.choice([3, 4, 8])
        sym = rng.random() < 0.5
        g = rng.choice([32, 64, 128])
        rows = rng.choice([1, 5, 32, 130])
        cols = g * rng.choice([1, 2, 4, 9]) if gran == 'per_group' else rng.choice([8, 100, 512, 1001])
        round_zp = rng.random() < 0.8
        osf = rng.choice([1, 1, 0.5, 1.7])
        gg = torch.Generator().manual_seed(rng.randrange(1 << 30))
        x = (torch.randn(rows, cols, generator=gg) * rng.choice([0.02, 1.0, 30.0])).to(dtype)
        calib = (torch.randn(rows, cols, generator=gg) * rng.choice([0.02, 1.0, 30.0])).to(dtype)
        kw = dict(group_size=g) if gran == 'per_group' else {}
        desc = f'draw {it}: {dtype} qparams {qp_dtype} {gran} w{bit} sym={sym} g={g} ({rows},{cols}) round_zp={round_zp} osf={osf}'
        spec = Q.IntSpec(bit, sym, gran, group_size=kw.get('group_size', 0), round_zp=round_zp)
        q = IntegerQuantizer(bit, sym, gran, round_zp=round_zp, **kw)
        _, s, z, qmax, qmin = Q.int_tensor_qparams(spec, calib)
        dimensioned = torch.is_tensor(z) and z.dim() > 0
        if s.dim() > 0:
            s = s.to(qp_dtype)
            z = z.to(qp_dtype) if dimensioned else z
        zd = z.to(dev) if dimensioned else z
        args = dict(scales=s.to(dev), zeros=zd, qmax=qmax, qmin=qmin, output_scale_factor=osf)
        if gran == 'per_token':
            got = q.fake_quant_act_static(x.to(dev), dict(scales=s.to(dev), zeros=zd, qmax=qmax, qmin=qmin))
            want = Q.int_fake_quant_static(spec, x, s, z, qmax, qmin)
        else:
            got = q.fake_quant_weight_static(x.to(dev), dict(args))
            want = Q.int_fake_quant_static(spec, x, s, z, qmax, qmin, output_scale_factor=osf)
        if not _same(got, want):
            problems.append(f'{desc}: fake quant, {_differing(got, want)}')
        if round_zp and gran != 'per_token':
            c, rs, _ = q.real_quant_weight_static(x.to(dev), dict(args))
            oc, ors, _ = Q.int_real_quant_static(spec, x, s, z, qmax, qmin, output_scale_factor=osf)
            if not (_same(c, oc) and _same(rs, ors)):
                problems.append(f'{desc}: real quant')
    assert not problems, '\n'.join(problems)


class _Layer:
    def __init__(self, w):
        self.weight = torch.nn.Parameter(w, requires_grad=False)


@pytest.mark.parametrize('seed', [0, 1])
def test_random_gptq_configs(dev, seed):
    """GPTQ of one Linear (gptq.py:96-245) with drawn bit width, group and block sizes (multiples of 128 and not),
    act-order, weight and activation types, both chains: the summed loss within 1 % of the oracle's."""
    from lightcompress_amd.gptq import GPTQ
    rng = random.Random(4000 + seed)
    problems, ran = [], 0
    while ran < 12:
        bit = rng.choice([2, 3, 4, 4, 8])
        sym = rng.random() < 0.4
        gran = rng.choice(['per_group', 'per_group', 'per_group', 'per_channel'])
        g = rng.choice([32, 64, 128, 128, 256, 100])
        bs = rng.choice([128, 128, 128, 64, 256, 100])
        K = rng.choice([256, 384, 512, 640, 1000, 1152])
        if gran == 'per_group' and K % g != 0:
            g = 128 if K % 128 == 0 else K // 4
        if gran == 'per_group' and K % g != 0:
            continue
        R = rng.choice([8, 24, 40, 130])
        actorder = rng.random() < 0.5
        wdtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        xdtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        block_factor = rng.random() < 0.7
        nb, T = rng.choice([(3, 200), (6, 96), (1, 700)])
        desc = (f'draw {ran}: w{bit} sym={sym} {gran} g={g} blocksize={bs} R={R} K={K} actorder={actorder} weight {wdtype} '
                f'activations {xdtype} block_factor={block_factor} {nb} x {T} tokens')
        ran += 1
        gg = torch.Generator().manual_seed(rng.randrange(1 << 30))
        sig = torch.exp(0.5 * torch.randn(K, generator=gg))
        batches = [(torch.randn(T, K, generator=gg) * sig).to(xdtype) for _ in range(nb)]
        w0 = (torch.randn(R, K, generator=gg) * 0.02).to(wdtype)
        spec = Q.IntSpec(bit, sym, gran, group_size=g if gran == 'per_group' else 0)
        h, n = torch.zeros(K, K), 0
        for b in batches:
            n = G.add_batch(h, n, b.unsqueeze(0))
        wcfg = dict(bit=bit, symmetric=sym, granularity=gran)
        if gran == 'per_group':
            wcfg['group_size'] = g
        gp = GPTQ({'weight': wcfg, 'special': dict(actorder=actorder, static_groups=False, percdamp=0.01, blocksize=bs,
                                                  true_sequential=True, block_factor=block_factor)})
        layer = _Layer(w0.to(dev))
        gp.collect_layer_qparams(layer)
        gp.subset_init({'layers': {'fc': layer}})
        for b in batches:
            gp.add_batch(layer, 'fc', b.unsqueeze(0).to(dev), None)
        gp.subset_transform({'layers': {'fc': layer}})
        loss = float(gp.last_errors['fc'])
        kw = {}
        if gran == 'per_channel':                          # the range of a whole row is fixed before the loop
            _, s0, z0, _, _ = Q.int_tensor_qparams(spec, w0)
            kw['static_qparams'] = (s0.float(), z0.float() if torch.is_tensor(z0) and z0.dim() > 0 else z0)
        ref = G.gptq_layer(w0, h, spec, blocksize=bs, actorder=actorder, **kw)
        if not bool(torch.isfinite(layer.weight.data).all()):
            problems.append(f'{desc}: weights not finite')
        elif not abs(loss - ref['loss']) <= 0.01 * ref['loss']:
            problems.append(f'{desc}: loss {loss:.6g}, oracle {ref["loss"]:.6g}')
    assert not problems, '\n'.join(problems)


@pytest.mark.parametrize('seed', [0, 1])
def test_random_awq_configs(dev, seed):
    """search_scale_subset (awq.py:178-278) against the oracle evaluated on GPU tensors (the inspect module then runs
    through the same GPU GEMMs on both sides): the 20 losses to 2e-5 relative, the same grid point unless two tie
    within that, and for 16-bit models the same scale bits (on these draws: the two means are fp32 sums in another
    order than torch's, and a sum next to a 16-bit rounding boundary can round the other way - about one scale in a
    thousand, none here).  fp32 models carry the summation order of mean|x| in the
    last place of every scale, which moves weights across rounding boundaries: their losses are held to 5e-3 (an 8-bit
    loss is a sum of few such events)."""
    from lightcompress_amd.awq import Awq
    rng = random.Random(5000 + seed)
    problems = []
    for it in range(24):
        dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        gran = rng.choice(['per_group', 'per_group', 'per_channel'])
        gs = rng.choice([32, 64, 128]) if gran == 'per_group' else 0
        K = rng.choice([128, 256, 384, 512, 1024])
        if gs and K % gs:
            K = gs * 4
        T, B = rng.choice([16, 50, 128, 300]), rng.choice([1, 2, 3])
        outs = [rng.choice([64, 96, 256, 520]) for _ in range(rng.choice([1, 2, 3]))]
        bit, sym = rng.choice([3, 4, 4, 8]), rng.choice([False, False, True])
        version = rng.choice(['v1', 'v2']) if gran == 'per_group' else 'v2'
        gg = torch.Generator().manual_seed(rng.randrange(1 << 30))
        sigma = torch.exp(torch.randn(K, generator=gg) * rng.choice([0.3, 1.0, 1.5]))
        x = (torch.randn(B, T, K, generator=gg) * sigma).to(dtype)
        ws = {f'w{i}': (torch.randn(o, K, generator=gg) * 0.02).to(dtype) for i, o in enumerate(outs)}
        desc = f'draw {it}: {dtype} {gran} g={gs} w{bit} sym={sym} {version} K={K} tokens {B}x{T} outputs {outs}'
        spec = Q.IntSpec(bit, sym, gran, group_size=gs)
        spec.qmin, spec.qmax = spec.qmin.to(dev), spec.qmax.to(dev)

        def forward(xx, ww):
            return torch.cat([xx @ w.t() for w in ww.values()], dim=-1)

        best_o, losses_o = A.search_scale({k: v.to(dev) for k, v in ws.items()}, x.to(dev), forward, spec, version=version)
        layers = {k: types.SimpleNamespace(weight=types.SimpleNamespace(data=v.to(dev))) for k, v in ws.items()}
        kw = dict(bit=bit, symmetric=sym, granularity=gran)
        if gs:
            kw['group_size'] = gs
        awq = Awq({'weight': kw, 'special': {'trans_version': version}})
        best = awq.search_scale_subset(None, layers, [x.to(dev)],
                                       lambda xx: torch.cat([xx @ l.weight.data.t() for l in layers.values()], dim=-1), False, {})
        losses, lo = awq.search_losses.cpu().double(), torch.tensor(losses_o).double()
        tol = 5e-3 if dtype == torch.float32 else (5e-5 if bit == 8 else 2e-5)     # (8-bit losses are rounding noise of the GEMMs)
        rel = float(((losses - lo).abs() / lo).max())
        if not rel <= tol:
            problems.append(f'{desc}: losses differ by {rel:.3g}')
        a, b = int(losses.argmin()), int(lo.argmin())
        if a != b:
            if abs(float(lo[a] - lo[b])) > tol * float(lo[b]):
                problems.append(f'{desc}: grid point {a} against {b}')
        elif dtype != torch.float32:
            if not _same(best, best_o):
                problems.append(f'{desc}: scales, {_differing(best, best_o)}')
        elif not torch.allclose(best.cpu(), best_o.cpu(), rtol=1e-5):
            problems.append(f'{desc}: fp32 scales')
    assert not problems, '\n'.join(problems)


@pytest.mark.parametrize('seed', [0])
def test_random_pack_configs(dev, seed):
    """The two on-disk layouts (module_utils.py:929-955, 1097-1158) on drawn shapes, types and data: AutoAWQ words, fp16
    scales and packed zero points from asymmetric 4-bit qparams; compressed-tensors words of symmetric 4 / 8-bit codes,
    also with a column count that does not fill the last word, and the fused quantize-and-pack."""
    from oracle import pack_ref as P
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.module_utils import AutoawqRealQuantLinear, VllmRealQuantLinear
    rng = random.Random(6000 + seed)
    problems = []
    for it in range(40):
        dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
        g = rng.choice([32, 64, 128])
        R, K = 32 * rng.choice([1, 2, 5, 9]), g * rng.choice([1, 2, 3, 8, 17])
        gg = torch.Generator().manual_seed(rng.randrange(1 << 30))
        w = (torch.randn(R, K, generator=gg) * rng.choice([0.02, 1.0, 50.0])).to(dtype)
        if rng.random() < 0.3:
            w[torch.rand(R, K, generator=gg) < 0.01] *= 30
        desc = f'draw {it}: {dtype} g={g} ({R},{K})'
        spec = Q.IntSpec(4, False, 'per_group', group_size=g)
        q = IntegerQuantizer(4, False, 'per_group', group_size=g)
        _, s, z = q.real_quant_weight_dynamic(w.to(dev))
        _, os_, oz = Q.int_real_quant_dynamic(spec, w)
        got = AutoawqRealQuantLinear.gemm_pack(None, w.to(dev), s, z, {'weight': dict(bit=4, group_size=g, pack_version='gemm_pack')})
        want = P.gemm_pack(w, os_, oz, g)
        if not all(_same(a, b) for a, b in zip(got, want)):
            problems.append(f'{desc}: AutoAWQ layout')
        for bit in (4, 8):
            kc = K if rng.random() < 0.5 else max(K - rng.choice([1, 3, 5]), 1)
            gran = 'per_channel' if kc != K else rng.choice(['per_group', 'per_channel'])
            kw = dict(group_size=g) if gran == 'per_group' else {}
            wc = w[:, :kc].contiguous()
            cspec = Q.IntSpec(bit, True, gran, group_size=kw.get('group_size', 0))
            cq = IntegerQuantizer(bit, True, gran, **kw)
            c, sc, _ = cq.real_quant_weight_dynamic(wc.to(dev))
            oc, osc, _ = Q.int_real_quant_dynamic(cspec, wc)
            want = P.pack_ct(oc, osc, bit)
            if not all(_same(a, b) for a, b in zip(VllmRealQuantLinear.pack(c, sc, {'weight': {'bit': bit}}), want)):
                problems.append(f'{desc}: compressed-tensors w{bit} {gran} K={kc}')
            if bit == 4 and gran == 'per_group':
                if not all(_same(a, b) for a, b in zip(VllmRealQuantLinear.quant_pack_fused(wc.to(dev), cq, {'weight': {'bit': 4}}), want)):
                    problems.append(f'{desc}: fused quantize and pack')
    assert not problems, '\n'.join(problems)
