"""GPU parity of the AWQ scale-search path against the CPU oracle."""
import types

import pytest
import torch

from oracle import awq_ref as A, quant_ref as Q
from tests.helpers import assert_bit_equal, gen
from tests.test_oracle_awq import swiglu, tiny_case

pytestmark = pytest.mark.gpu

CFG = {'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128), 'special': {}}


def make_awq(**special):
    from lightcompress_amd.awq import Awq
    return Awq({'weight': dict(CFG['weight']), 'special': special})


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize('shape', [(256, 512), (1000, 1024), (96, 4096)])
def test_scale_quant_bit_exact(dev, dtype, shape):
    R, K = shape
    w = (torch.randn(R, K, generator=gen(1)) * 0.02).to(dtype)
    s = torch.exp(torch.randn(K, generator=gen(2)) * 0.5).to(dtype)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    got = make_awq()._scale_quant(w.to(dev), s.to(dev))
    assert_bit_equal(got, A.scale_and_fake_quant(w, s, spec), 'W*s -> fake quant')
    wd = w.to(dev)
    fc = types.SimpleNamespace(weight=types.SimpleNamespace(data=wd))
    make_awq().fake_quantize_weight(fc, s.to(dev), False, 'fc')
    assert_bit_equal(fc.weight.data, A.scale_and_fake_quant(w, s, spec), 'fake_quantize_weight')
    assert torch.equal(wd.cpu(), w)                                # the caller's tensor is left alone


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32, torch.float16])
def test_scaling_input_bit_exact(dev, dtype):
    x = (torch.randn(3, 100, 1024, generator=gen(3)) * 2).to(dtype)
    s = torch.exp(torch.randn(1024, generator=gen(4)) * 0.5).to(dtype)
    assert_bit_equal(make_awq().scaling_input(x.to(dev), s.to(dev), False), A.scaling_input(x, s), 'x / s')


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32, torch.float16])
def test_act_scale_weight_scale_and_loss(dev, dtype):
    x, w, down = tiny_case(dtype, seed=5, T=300, K=512, I=640)
    awq = make_awq()
    awq._bs = x.shape[0]
    got = awq.get_act_scale(x.to(dev)).cpu()
    want = A.act_scale(x)
    assert got.dtype == dtype
    # the sum order differs from torch's: compare before the final rounding to the tensor type
    ref64 = x.double().abs().reshape(-1, 512).mean(0)
    tol = {torch.bfloat16: 2 ** -8, torch.float16: 2 ** -11, torch.float32: 1e-6}[dtype]
    assert float(((got.double() - ref64).abs() / ref64).max()) <= tol
    if dtype == torch.bfloat16:                                     # after rounding to bf16 almost all entries coincide
        assert float((got.float() != want.float()).float().mean()) < 0.02
    layers = {k: types.SimpleNamespace(weight=types.SimpleNamespace(data=v.to(dev))) for k, v in w.items()}
    ws = awq.get_weight_scale(layers).cpu()
    wo = A.weight_scale(list(w.values()), Q.IntSpec(4, False, 'per_group', group_size=128))
    assert float(((ws.double() - wo.double()).abs() / wo.double()).max()) <= 2 * tol
    a = (torch.randn(4, 64, 512, generator=gen(6))).to(dtype)
    b = (a.float() + torch.randn(4, 64, 512, generator=gen(7)) * 0.1).to(dtype)
    l = awq.calculate_loss(a.to(dev), b.to(dev))
    assert abs(l - A.loss(a, b)) <= 1e-5 * A.loss(a, b)


class Fc:
    def __init__(self, w):
        self.weight = types.SimpleNamespace(data=w)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_search_scale_subset_picks_the_oracle_ratio(dev, dtype):
    x, w, down = tiny_case(dtype, seed=8, T=256, K=512, I=768)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: swiglu(xx, dict(ww, down=down))
    best_o, losses_o = A.search_scale(w, x, fwd, spec)
    layers = {k: Fc(v.to(dev)) for k, v in w.items()}
    downd = down.to(dev)
    inspect = lambda xx: swiglu(xx, {'gate': layers['gate'].weight.data, 'up': layers['up'].weight.data, 'down': downd})
    awq = make_awq()
    best = awq.search_scale_subset(None, layers, [x.to(dev)], inspect, False, {})
    losses = awq.search_losses.cpu()
    assert best.dtype == dtype and best.shape == (512,)
    rel = ((losses.double() - torch.tensor(losses_o).double()).abs() / torch.tensor(losses_o).double()).max()
    assert float(rel) < {torch.bfloat16: 0.05, torch.float16: 0.01, torch.float32: 1e-3}[dtype], float(rel)
    ko = min(range(20), key=lambda i: losses_o[i])
    kg = int(torch.argmin(losses))
    # GEMM rounding differs between CPU and GPU libraries; the chosen grid point may move only between near-ties
    assert kg == ko or abs(losses_o[kg] - losses_o[ko]) <= 0.02 * losses_o[ko]
    if kg == ko:
        assert float((best.cpu().float() - best_o.float()).abs().max()) <= 2 ** -7 * float(best_o.float().abs().max())
    # weights are back to the originals
    assert torch.equal(layers['gate'].weight.data.cpu(), w['gate'])


def test_search_scale_subset_gqa(dev):
    """v_proj -> o_proj with grouped query heads (is_gqa): scales from mean|v_proj(x)|, repeated per group."""
    dtype = torch.bfloat16
    kvh, hd, groups = 2, 64, 4                                    # o_proj sees 8 heads x 64 = 512 columns
    K = kvh * groups * hd
    g = gen(31)
    x = (torch.randn(2, 128, K, generator=g) * torch.exp(0.5 * torch.randn(K, generator=g))).to(dtype)
    wo = (torch.randn(384, K, generator=g) * 0.02).to(dtype)
    wv = (torch.randn(kvh * hd, K, generator=g) * 0.05).to(dtype)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: xx @ ww['o'].t()
    best_o, losses_o = A.search_scale({'o': wo}, x, fwd, spec, gqa=(lambda t: t @ wv.t(), kvh, hd, groups))
    awq = make_awq()
    awq.set_model_config(types.SimpleNamespace(hidden_size=K, num_attention_heads=kvh * groups, num_key_value_heads=kvh))
    assert awq.has_gqa and awq.head_dim == hd and awq.num_key_value_groups == groups
    layers = {'o': Fc(wo.to(dev))}
    wvd = wv.to(dev)
    best = awq.search_scale_subset(lambda t: t @ wvd.t(), layers, [x.to(dev)], lambda xx: xx @ layers['o'].weight.data.t(), True, {})
    losses = awq.search_losses.cpu()
    assert best.shape == (kvh * hd,) and best.dtype == dtype
    rel = ((losses.double() - torch.tensor(losses_o).double()).abs() / torch.tensor(losses_o).double()).max()
    assert float(rel) < 0.05, float(rel)
    ko, kg = min(range(20), key=lambda i: losses_o[i]), int(torch.argmin(losses))
    assert kg == ko or abs(losses_o[kg] - losses_o[ko]) <= 0.02 * losses_o[ko]
    if kg == ko:
        assert float((best.cpu().float() - best_o.float()).abs().max()) <= 2 ** -6 * float(best_o.float().abs().max())
    # the pieces, bit for bit: repeated scales on the weight and on the input
    s_kv = best_o
    rep = A.repeat_gqa(s_kv, kvh, hd, groups)
    assert_bit_equal(awq.scaling_input(x.to(dev), s_kv.to(dev), True), A.scaling_input(x, rep), 'x / repeated scales')
    fc = Fc(wo.to(dev).clone())
    assert_bit_equal(awq.fake_quantize_weight(fc, s_kv.to(dev), True, 'o').data, A.scale_and_fake_quant(wo, rep, spec),
                     'W * repeated scales -> fake quant')
    w2 = wo.to(dev).clone()
    assert_bit_equal(awq.scaling_weight(w2, s_kv.to(dev), True), wo * rep.view(1, -1), 'scaling_weight')


def _search_on_gpu(dev, awq, w, down, inputs):
    layers = {k: Fc(v.to(dev)) for k, v in w.items()}
    downd = down.to(dev)
    inspect = lambda xx: swiglu(xx, {'gate': layers['gate'].weight.data, 'up': layers['up'].weight.data, 'down': downd})
    best = awq.search_scale_subset(None, layers, [x.to(dev) for x in inputs], inspect, False, {})
    for k in w:
        assert torch.equal(layers[k].weight.data.cpu(), w[k])              # weights are back to the originals
    return best, awq.search_losses.cpu()


def _same_point(losses, losses_o, tol=0.02):
    ko = min(range(20), key=lambda i: losses_o[i])
    kg = int(torch.argmin(losses))
    return kg == ko, (kg == ko or abs(losses_o[kg] - losses_o[ko]) <= tol * losses_o[ko])


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_search_scale_subset_trans_version_v1(dev, dtype):
    """trans_version v1 (awq.py:97-102): scales = mean|x|^r / w_max^(1-r), w_max from get_weight_scale."""
    x, w, down = tiny_case(dtype, seed=18, T=192, K=512, I=640)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: swiglu(xx, dict(ww, down=down))
    best_o, losses_o = A.search_scale(w, x, fwd, spec, version='v1')
    best, losses = _search_on_gpu(dev, make_awq(trans_version='v1'), w, down, [x])
    rel = ((losses.double() - torch.tensor(losses_o).double()).abs() / torch.tensor(losses_o).double()).max()
    assert float(rel) < {torch.bfloat16: 0.05, torch.float16: 0.01, torch.float32: 1e-3}[dtype], float(rel)
    same, near = _same_point(losses, losses_o)
    assert near
    if same:
        assert float((best.cpu().float() - best_o.float()).abs().max()) <= 2 ** -6 * float(best_o.float().abs().max())
    # v1 and v2 really differ on this case
    _, losses_v2 = A.search_scale(w, x, fwd, spec, version='v2')
    assert max(abs(a - b) / b for a, b in zip(losses_o[1:], losses_v2[1:])) > 1e-3


@pytest.mark.parametrize('bs', [None, 1])
def test_search_scale_subset_several_inputs_and_micro_batches(dev, bs):
    """len(input) > 1 and awq_bs: the reference compares `loss_mean` after every input (awq.py:245-248), so the first
    input's loss picks the grid point and the returned scales are the mean over the inputs at that point."""
    dtype = torch.float32
    x0, w, down = tiny_case(dtype, seed=21, T=96, K=512, I=640)
    g = gen(22)
    x1 = (torch.randn(4, 96, 512, generator=g) * torch.exp(torch.randn(512, generator=g))).to(dtype)
    x2 = (torch.randn(2, 96, 512, generator=g) * 3).to(dtype)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    fwd = lambda xx, ww: swiglu(xx, dict(ww, down=down))
    inputs = [x0, x1, x2]
    best_o, trace = A.search_scale_inputs(w, inputs, fwd, spec, bs=bs)
    first = [row[0] for row in trace]
    special = {} if bs is None else {'awq_bs': bs}
    best, losses = _search_on_gpu(dev, make_awq(**special), w, down, inputs)
    rel = ((losses.double() - torch.tensor(first).double()).abs() / torch.tensor(first).double()).max()
    assert float(rel) < 1e-3, float(rel)
    same, near = _same_point(losses, first)
    assert near
    if same:
        assert float((best.cpu() - best_o).abs().max()) <= 1e-5 * float(best_o.abs().max())
    # the documented alternative: the mean loss over all inputs
    best_m, losses_m = _search_on_gpu(dev, make_awq(multi_input_select='mean', **special), w, down, inputs)
    full = [row[-1] for row in trace]
    rel = ((losses_m.double() - torch.tensor(full).double()).abs() / torch.tensor(full).double()).max()
    assert float(rel) < 1e-3, float(rel)


def test_search_honours_the_weight_quantizer_settings(dev):
    """fake_quantize_weight is wquantizer.fake_quant_weight_dynamic (awq.py:156): calib_algo mse and round_zp False
    change the quantized weights the loss is measured on."""
    from lightcompress_amd.awq import Awq
    from lightcompress_amd import IntegerQuantizer
    dtype = torch.float32
    w = (torch.randn(96, 512, generator=gen(41)) * 0.02).to(dtype)
    s = torch.exp(torch.randn(512, generator=gen(42)) * 0.5).to(dtype)
    for kw, spec_kw in (({'round_zp': False}, {'round_zp': False}), ({'calib_algo': 'mse'}, {})):
        cfg = {'weight': dict(CFG['weight'], **kw), 'special': {}}
        got = Awq(cfg)._scale_quant(w.to(dev), s.to(dev))
        spec = Q.IntSpec(4, False, 'per_group', group_size=128, **spec_kw)
        ws = w.clone().mul_(s.view(1, -1))
        if 'calib_algo' in kw:
            rows = Q.reshape_rows(spec, ws)
            lo, hi = Q.int_mse_range(spec, rows)
            sc, zp, qmax, qmin = Q.int_qparams(spec, lo, hi)
            want = Q.int_quant_dequant(spec, rows, sc, zp, qmax, qmin).reshape(ws.shape)
            assert float((got.cpu() == want).float().mean()) > 0.98        # the shrink search may tie between steps
        else:
            assert_bit_equal(got, Q.int_fake_quant_dynamic(spec, ws), 'round_zp False')
        plain = make_awq()._scale_quant(w.to(dev), s.to(dev))
        assert not torch.equal(plain, got)


def test_search_on_float8_blockwise_weights(dev):
    """A block-wise float8 checkpoint (awq.py:53-56, 148-162): bf16 <- weight * weight_scale_inv, scale, fake quant,
    cast back to float8 with fresh block scales; weight and weight_scale_inv are both restored after the search."""
    x, w, down = tiny_case(torch.bfloat16, seed=25, T=128, K=512, I=640)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)

    class Fp8Fc:
        def __init__(self, wt):
            y, sc = Q.triton_weight_cast_to_fp8(wt)
            self.weight = types.SimpleNamespace(data=y.to(dev))
            self.weight_scale_inv = types.SimpleNamespace(data=sc.to(dev))
    layers = {k: Fp8Fc(v) for k, v in w.items()}
    w8 = {k: (layers[k].weight.data.cpu(), layers[k].weight_scale_inv.data.cpu()) for k in w}
    wb = {k: Q.triton_weight_cast_to_bf16(*w8[k]).to(torch.bfloat16) for k in w}
    awq = make_awq()
    # one grid point's weight, bit for bit
    s = torch.exp(torch.randn(512, generator=gen(26)) * 0.3).bfloat16()
    fc = Fp8Fc(w['gate'])
    awq.fake_quantize_weight(fc, s.to(dev), False, 'gate')
    yo, so = Q.triton_weight_cast_to_fp8(A.scale_and_fake_quant(wb['gate'], s, spec))
    assert_bit_equal(fc.weight.data.view(torch.uint8), yo.view(torch.uint8), 'float8 codes')
    assert_bit_equal(fc.weight_scale_inv.data, so, 'block scales')
    # get_weight_scale sees the bf16 weights
    ws = awq.get_weight_scale(layers).cpu()
    wo = A.weight_scale(list(wb.values()), spec)
    assert float(((ws.double() - wo.double()).abs() / wo.double()).max()) <= 2 ** -7
    # the search: the inspect module dequantises what the layers hold
    downd = down.to(dev)
    def deq(fc):
        from lightcompress_amd.kernel import weight_cast_to_bf16
        return weight_cast_to_bf16(fc.weight.data, fc.weight_scale_inv.data).to(torch.bfloat16)
    inspect = lambda xx: swiglu(xx, {'gate': deq(layers['gate']), 'up': deq(layers['up']), 'down': downd})
    def fwd(xx, ww):
        q = {k: Q.triton_weight_cast_to_bf16(*Q.triton_weight_cast_to_fp8(v)).to(torch.bfloat16) if ww is not wb else v
             for k, v in ww.items()}
        return swiglu(xx, dict(q, down=down))
    best_o, losses_o = A.search_scale(wb, x, fwd, spec)
    best = awq.search_scale_subset(None, layers, [x.to(dev)], inspect, False, {})
    losses = awq.search_losses.cpu()
    rel = ((losses.double() - torch.tensor(losses_o).double()).abs() / torch.tensor(losses_o).double()).max()
    assert float(rel) < 0.05, float(rel)
    assert _same_point(losses, losses_o)[1]
    for k in w:
        assert torch.equal(layers[k].weight.data.cpu().view(torch.uint8), w8[k][0].view(torch.uint8))
        assert torch.equal(layers[k].weight_scale_inv.data.cpu(), w8[k][1])


# ---- AutoClipper (auto_clip.py) ---------------------------------------------------------------------
@pytest.mark.parametrize('clip_sym,sym', [(False, False), (True, False), (False, True)])
@pytest.mark.parametrize('R,K,T', [(64, 256, 96), (320, 512, 512), (256, 128, 700)])
def test_auto_clip_mfma_kernel_against_oracle(dev, clip_sym, sym, R, K, T):
    """AutoClipper.fast = True.  Errors of the ten shrink steps within the bf16 noise of the reference's chain (it rounds both dot products
    to bf16 before subtracting; the kernel multiplies the weight difference on MFMA), the same step chosen wherever
    the oracle's own errors separate the best two by more than 3 %, ranges identical there."""
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.auto_clip import AutoClipper
    from tests.helpers import weight_like
    spec = Q.IntSpec(4, sym, 'per_group', group_size=128)
    w = weight_like(R, K, seed=R + K, dtype=torch.bfloat16)
    x = (torch.randn(T, K, generator=gen(R + T)) * torch.exp(0.5 * torch.randn(K, generator=gen(K + T)))).bfloat16()
    nst = 512
    obmax, obmin, oerrs = A.auto_clip_layer(spec, w, [x.clone()], clip_sym=clip_sym, n_sample_token=nst)
    wq = IntegerQuantizer(4, sym, 'per_group', group_size=128)
    clipper = AutoClipper(True, wq, None, 'v1', clip_sym, False, None)
    clipper.fast = True
    bmax, bmin = clipper.auto_clip_layer(0, 'fc', w.to(dev), [x.to(dev)], n_sample_token=nst)
    assert bmax.shape == obmax.shape and bmin.shape == obmin.shape and bmax.dtype == torch.bfloat16
    errs = clipper.last_errs.cpu()
    rel = (errs.double() - oerrs.double()).abs() / oerrs.double().clamp(min=1e-30)
    assert float(rel.median()) < 0.02 and float(rel.quantile(0.99)) < 0.25
    top2 = oerrs.float().topk(2, dim=-1, largest=False).values
    clear = (top2[..., 1] > 1.03 * top2[..., 0]).unsqueeze(-1)
    assert float(clear.float().mean()) > 0.3
    assert torch.equal(bmax.cpu()[clear], obmax[clear]) and torch.equal(bmin.cpu()[clear], obmin[clear])
    assert float((bmax.cpu() == obmax).float().mean()) > 0.9
    # every answer is one of the shrunken original ranges
    wg = w.reshape(R, K // 128, 128)
    org = (wg.abs().amax(-1) if clip_sym else wg.amax(-1)).unsqueeze(-1)
    cands = torch.cat([org * (1 - s / 20) for s in range(10)], dim=-1)
    assert bool((bmax.cpu() == cands).any(-1).all())
    # apply_clip clamps the layer weight group-wise
    layer = torch.nn.Linear(K, R, bias=False, dtype=torch.bfloat16, device=dev)
    layer.weight.data.copy_(w)
    clipper.apply_clip(0, layer, bmin, bmax, 'fc')
    assert_bit_equal(layer.weight.data, A.apply_clip_v1(w, bmin.cpu(), bmax.cpu(), clip_sym), 'apply_clip')


_CLIP_CASES = [
    # version, w_only, weight spec (bit, sym, granularity, group), clip_sym, dtype, R, K, token counts of the inputs
    ('v1', True, (4, False, 'per_group', 128), False, torch.bfloat16, 320, 512, [512]),
    ('v1', True, (4, False, 'per_group', 128), True, torch.bfloat16, 64, 256, [96]),
    ('v1', True, (4, True, 'per_group', 64), False, torch.bfloat16, 128, 320, [200, 75]),
    ('v1', True, (3, False, 'per_group', 32), False, torch.float32, 64, 96, [130]),
    ('v1', True, (4, False, 'per_channel', 0), False, torch.bfloat16, 64, 300, [64]),
    ('v1', False, (4, False, 'per_group', 128), False, torch.bfloat16, 256, 256, [300]),
    ('v2', False, (8, True, 'per_channel', 0), True, torch.bfloat16, 64, 384, [100]),
    ('v2', True, (4, False, 'per_channel', 0), False, torch.float32, 64, 256, [80, 80]),
    ('v2', False, (4, False, 'per_group', 128), False, torch.bfloat16, 64, 256, [64]),
    ('v1', True, (4, False, 'per_group', 128), False, torch.float16, 128, 512, [256]),
    ('v1', False, (4, True, 'per_group', 64), True, torch.float16, 64, 256, [100, 60]),
    ('v2', True, (4, False, 'per_channel', 0), False, torch.float16, 64, 256, [80]),
]


@pytest.mark.parametrize('ver,w_only,wspec,clip_sym,dtype,R,K,Ts', _CLIP_CASES)
def test_auto_clip_reference_rounding_sequence(dev, ver, w_only, wspec, clip_sym, dtype, R, K, Ts):
    """The default search path against the op-for-op oracle: the same products rounded to the tensors' type, the same
    rounded sums, difference, square and mean.  What is left is the order of the fp32 additions inside a group sum
    and inside the mean over tokens (torch's reduction order on the CPU differs from the kernel's): a sum that lands
    within 1e-7 of a rounding boundary may round the other way.  Bar (bf16): at least 99 % of the 10 errors per (row,
    group) identical bit for bit, every error within two units of its last place (fp32: within 5e-4 relative), the same range on at least 99 % of the
    groups, and wherever the range differs the oracle's own error of the step chosen here is within two units of
    the last place of its minimum (a tie at the precision of the comparison)."""
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.auto_clip import AutoClipper
    from tests.helpers import weight_like
    bit, sym, gran, g = wspec
    spec = Q.IntSpec(bit, sym, gran, group_size=g)
    aspec = None if w_only else Q.IntSpec(8, True, 'per_token')
    w = weight_like(R, K, seed=R + K, dtype=dtype)
    xs = [(torch.randn(T, K, generator=gen(R + T + i)) * torch.exp(0.5 * torch.randn(K, generator=gen(K + T)))).to(dtype)
          for i, T in enumerate(Ts)]
    nst = 128
    obmax, obmin, oerrs = A.auto_clip_layer(spec, w, [x.clone() for x in xs], clip_sym=clip_sym, n_sample_token=nst,
                                            clip_version=ver, aspec=aspec)
    wq = IntegerQuantizer(bit, sym, gran, group_size=g) if gran == 'per_group' else IntegerQuantizer(bit, sym, gran)
    aq = None if w_only else IntegerQuantizer(8, True, 'per_token')
    clipper = AutoClipper(w_only, wq, aq, ver, clip_sym, True, None)
    bmax, bmin = clipper.auto_clip_layer(0, 'fc', w.to(dev), [x.to(dev) for x in xs], n_sample_token=nst)
    assert bmax.shape == obmax.shape and bmin.shape == obmin.shape and bmax.dtype == dtype
    errs, oe = clipper.last_errs.cpu().double(), oerrs.double()
    # fp32 tensors round nothing away: there the summation order shows in every error (cancellation in out - org)
    ulp = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10, torch.float32: 2.5e-4}[dtype]
    if dtype != torch.float32:
        same = ((errs == oe) | (errs.isnan() & oe.isnan())).float().mean()
        assert float(same) > 0.99, float(same)
    fin = oe.isfinite()
    floor = 2.0 ** -24 if dtype == torch.float16 else 0.0      # fp16: small errors are subnormal, their last place is 2^-24
    assert bool(((errs - oe).abs()[fin] <= 2 * torch.clamp(ulp * oe.abs()[fin], min=floor)).all())
    eq = (bmax.cpu() == obmax) & (bmin.cpu() == obmin)
    assert float(eq.float().mean()) > 0.99, float(eq.float().mean())
    if not bool(eq.all()):
        G = obmax.shape[1]
        hi0 = (w.reshape(R, G, -1).abs().amax(-1) if clip_sym else w.reshape(R, G, -1).amax(-1)).unsqueeze(-1)
        cands = torch.cat([hi0 * (1 - s / 20) for s in range(10)], dim=-1)
        step = (cands == bmax.cpu()).float().argmax(-1)
        picked = oe.gather(-1, step.unsqueeze(-1)).squeeze(-1)
        best = oe.min(-1).values
        bad = ~eq.squeeze(-1)
        assert bool((picked[bad] <= best[bad] * (1 + 4 * ulp) + 4 * floor).all())
    # apply_clip: v1 clamps the weight group-wise, v2 stores the sigmoid factors of the found range
    layer = torch.nn.Linear(K, R, bias=False, dtype=dtype, device=dev)
    layer.weight.data.copy_(w)
    clipper.apply_clip(3, layer, bmin, bmax, 'fc')
    if ver == 'v1':
        assert_bit_equal(layer.weight.data, A.apply_clip_v1(w, bmin.cpu(), bmax.cpu(), clip_sym), 'apply_clip')
    else:
        up, low = A.clip_factor(spec, w, bmin.cpu(), bmax.cpu(), clip_sym)
        tol = dict(rtol=2e-2, atol=2e-2) if dtype != torch.float32 else dict(rtol=1e-4, atol=1e-5)
        got_up = layer.buf_upbound_factor.cpu()
        fin = up.isfinite()
        assert got_up.shape == up.shape and torch.equal(got_up.isfinite(), fin)
        assert torch.allclose(got_up[fin].float(), up[fin].float(), **tol)
        assert (layer.buf_lowbound_factor is None) == (low is None)
        assert clipper.weight_clips[3]['fc.weight_quantizer.upbound_factor'].shape == up.shape
        # the stored factors drive calib_algo='learnable' (quant.py:207-221) to the clipped quantization
        lq = IntegerQuantizer(bit, sym, gran, group_size=g, calib_algo='learnable') if gran == 'per_group' else \
            IntegerQuantizer(bit, sym, gran, calib_algo='learnable')
        args = {'upbound_factor': layer.buf_upbound_factor, 'lowbound_factor': layer.buf_lowbound_factor}
        got = lq.fake_quant_weight_dynamic(layer.weight.data, args)
        # sigmoid comes from two math libraries (GPU / CPU torch): the range within an ulp of the oracle's, then the
        # quantization of the oracle on the GPU's range bit for bit
        lo_g, hi_g = lq.get_learnable_range(lq.reshape_tensor(layer.weight.data), **args)
        lo_l, hi_l = A.learnable_range(spec, Q.reshape_rows(spec, w), None if low is None else layer.buf_lowbound_factor.cpu(),
                                       got_up)
        rt = 1e-2 if dtype != torch.float32 else 1e-6
        assert torch.allclose(hi_g.cpu().float(), hi_l.float(), rtol=rt) and torch.allclose(lo_g.cpu().float(), lo_l.float(), rtol=rt)
        sc, z, qmax, qmin = Q.int_qparams(spec, lo_g.cpu(), hi_g.cpu())
        want = Q.int_fake_quant_static(spec, w, sc, z, qmax, qmin)
        assert_bit_equal(got, want, 'learnable fake quant')


def test_auto_clip_run_skips_query_key_and_handles_float8_weights(dev):
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.auto_clip import AutoClipper
    from lightcompress_amd.kernel import weight_cast_to_fp8
    wq = IntegerQuantizer(4, False, 'per_group', group_size=128)
    blk = torch.nn.ModuleDict({'q_proj': torch.nn.Linear(128, 64, bias=False), 'o_proj': torch.nn.Linear(128, 64, bias=False)})
    blk = blk.to(device=dev, dtype=torch.bfloat16)
    q0, o0 = blk['q_proj'].weight.data.clone(), blk['o_proj'].weight.data.clone()
    x = torch.randn(4, 32, 128, generator=gen(5)).bfloat16().to(dev)
    AutoClipper(True, wq, None, 'v1', False, False, None).run(blk, 0, {'q_proj': [x], 'o_proj': [x[:2], x[2:]]}, 512)
    assert torch.equal(blk['q_proj'].weight.data, q0)                    # names with q_/k_ are not clipped
    assert not torch.equal(blk['o_proj'].weight.data, o0)
    assert float((blk['o_proj'].weight.data.abs() <= o0.abs()).float().mean()) == 1.0
    # v2 registers the factor buffers, None on the skipped layers
    blk['o_proj'].weight.data.copy_(o0)
    AutoClipper(True, wq, None, 'v2', False, False, None).run(blk, 0, {'q_proj': [x], 'o_proj': [x]}, 512)
    assert blk['q_proj'].buf_upbound_factor is None and blk['o_proj'].buf_upbound_factor.shape == (64, 1)
    assert torch.equal(blk['o_proj'].weight.data, o0)                    # v2 leaves the weight alone
    with pytest.raises(NotImplementedError):
        AutoClipper(True, IntegerQuantizer(4, False, 'per_tensor'), None, 'v1', False, False, None).auto_clip_layer(0, 'o', o0, [x])
    # a block-wise float8 layer is searched on its bf16 weights and cast back (auto_clip.py:48-81)
    fp8 = torch.nn.Linear(256, 128, bias=False).to(device=dev, dtype=torch.bfloat16)
    w8, s8 = weight_cast_to_fp8(fp8.weight.data.contiguous())
    fp8.weight.data = w8
    fp8.register_buffer('weight_scale_inv', s8)
    xb = torch.randn(64, 256, generator=gen(6)).bfloat16().to(dev)
    AutoClipper(True, wq, None, 'v1', False, False, None).run(torch.nn.ModuleDict({'o_proj': fp8}), 0, {'o_proj': [xb]}, 512)
    assert fp8.weight.data.dtype == torch.float8_e4m3fn and fp8.weight_scale_inv.shape == s8.shape
    assert bool((fp8.weight_scale_inv <= s8).all()) and bool(fp8.weight_scale_inv.isfinite().all())


# ---- apply_scale / scale_fc_fc / scale_ln_fcs / update_input_feat ---------------------------------------
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32, torch.float16])
def test_scale_folding_matches_the_torch_op_sequence(dev, dtype):
    """base_blockwise_quantization.py:619-723, 772-801, 899-920: each is a literal in-place torch op in the
    reference (one IEEE multiply / divide per element in the tensor's type), so the CPU op is the oracle: bit-exact."""
    from lightcompress_amd.blockwise import ScaleFolding
    sf = ScaleFolding()
    K, I = 256, 384
    s = (torch.rand(K, generator=gen(1)) + 0.5).to(dtype)
    def lin(i, o, bias, seed):
        m = torch.nn.Linear(i, o, bias=bias, dtype=torch.float32)
        m.weight.data = (torch.randn(o, i, generator=gen(seed)) * 0.05)
        if bias:
            m.bias.data = torch.randn(o, generator=gen(seed + 1)) * 0.05
        return m.to(dtype)
    # ln -> fcs
    ln = torch.nn.LayerNorm(K, dtype=dtype)
    ln.weight.data = (torch.rand(K, generator=gen(2)) + 0.5).to(dtype); ln.bias.data = torch.randn(K, generator=gen(3)).to(dtype)
    fcs = [lin(K, I, False, 10), lin(K, I, True, 20)]
    want_lnw, want_lnb = ln.weight.data / s, ln.bias.data / s
    want_fc = [fc.weight.data * s.view(1, -1) for fc in fcs]
    ln_d = ln.to(dev); fcs_d = [fc.to(dev) for fc in fcs]
    sf.apply_scale(s.to(dev), [ln_d], fcs_d)
    assert_bit_equal(ln_d.weight.data, want_lnw, 'ln weight'); assert_bit_equal(ln_d.bias.data, want_lnb, 'ln bias')
    for fc, wnt in zip(fcs_d, want_fc):
        assert_bit_equal(fc.weight.data, wnt, 'fc weight')
    # fc -> fc, equal widths (with bias) and the gated case (fc1 twice as wide)
    s2 = (torch.rand(I, generator=gen(4)) + 0.5).to(dtype)
    for mult in (1, 2):
        fc1, fc2 = lin(K, I * mult, True, 30 + mult), lin(I, K, False, 40 + mult)
        w1, b1, w2 = fc1.weight.data.clone(), fc1.bias.data.clone(), fc2.weight.data.clone()
        if mult == 1:
            w1 = w1 / s2.view(-1, 1); b1 = b1 / s2
        else:
            w1[I:] = w1[I:] / s2.view(-1, 1); b1[I:] = b1[I:] / s2
        w2 = w2 * s2.view(1, -1)
        f1, f2 = fc1.to(dev), fc2.to(dev)
        sf.apply_scale(s2.to(dev), [f1], [f2])
        assert_bit_equal(f1.weight.data, w1, 'fc1 weight'); assert_bit_equal(f1.bias.data, b1, 'fc1 bias')
        assert_bit_equal(f2.weight.data, w2, 'fc2 weight')
    # cached inputs
    x = torch.randn(3, 40, K, generator=gen(5)).to(dtype)
    feat = {'a': [x[:2].to(dev), x[2:].to(dev)]}
    sf.update_input_feat(s.to(dev), feat, {'a': None}, False)
    assert_bit_equal(torch.cat(feat['a']), x / s.view(1, -1), 'scaled inputs')
    # fused QKV, output channels laid out [head][q, k, v][head_dim] (:648-676): the reference's transposed reshapes,
    # written here as an index loop - only value rows change, row (h, 2, d) by scales[h * hd + d]
    heads, hd = 6, I // 6
    sf.num_heads = heads
    fc1, fc2 = lin(K, 3 * I, True, 50), lin(I, K, False, 51)
    w1, b1, w2 = fc1.weight.data.clone(), fc1.bias.data.clone(), fc2.weight.data.clone()
    for h in range(heads):
        for d in range(hd):
            o = (h * 3 + 2) * hd + d
            w1[o] = w1[o] / s2[h * hd + d]
            b1[o] = b1[o] / s2[h * hd + d]
    w2 = w2 * s2.view(1, -1)
    f1, f2 = fc1.to(dev), fc2.to(dev)
    sf.scale_fc_fc(f1, f2, s2.to(dev))
    assert_bit_equal(f1.weight.data, w1, 'fused qkv weight'); assert_bit_equal(f1.bias.data, b1, 'fused qkv bias')
    assert_bit_equal(f2.weight.data, w2, 'fc2 after fused qkv')


def test_scale_folding_float8_blockwise_weights(dev):
    """Float8 block-wise checkpoints (:690-699, 711-720, 786-793): bf16 <- weight * weight_scale_inv, scale, cast back.
    Oracle = the block-wise cast oracles around the literal bf16 torch op."""
    from lightcompress_amd.blockwise import ScaleFolding
    sf = ScaleFolding()
    K, I = 256, 384
    s = (torch.rand(I, generator=gen(61)) + 0.5).bfloat16()
    class Fp8Linear(torch.nn.Module):
        def __init__(self, i, o, seed):
            super().__init__()
            w = (torch.randn(o, i, generator=gen(seed)) * 0.05).bfloat16()
            y, sc = Q.triton_weight_cast_to_fp8(w)
            self.in_features, self.out_features, self.bias = i, o, None
            self.weight = torch.nn.Parameter(y, requires_grad=False)
            self.weight_scale_inv = torch.nn.Parameter(sc, requires_grad=False)
    fp8_linear = Fp8Linear
    to_dev = lambda m: m.to(dev)
    fc1, fc2 = fp8_linear(K, I, 70), fp8_linear(I, K, 71)
    t1 = Q.triton_weight_cast_to_bf16(fc1.weight.data, fc1.weight_scale_inv.data).to(torch.bfloat16)
    t1.div_(s.view(-1, 1))
    w1, sc1 = Q.triton_weight_cast_to_fp8(t1)
    t2 = Q.triton_weight_cast_to_bf16(fc2.weight.data, fc2.weight_scale_inv.data).to(torch.bfloat16)
    t2.mul_(s.view(1, -1))
    w2, sc2 = Q.triton_weight_cast_to_fp8(t2)
    ln = torch.nn.LayerNorm(I, dtype=torch.bfloat16)
    fc3 = fp8_linear(I, K, 72)
    t3 = Q.triton_weight_cast_to_bf16(fc3.weight.data, fc3.weight_scale_inv.data).to(torch.bfloat16)
    t3.mul_(s.view(1, -1))
    w3, sc3 = Q.triton_weight_cast_to_fp8(t3)
    f1, f2, f3 = to_dev(fc1), to_dev(fc2), to_dev(fc3)
    sf.scale_ln_fcs(ln.to(dev), [f3], s.to(dev))
    assert_bit_equal(f3.weight.data.view(torch.uint8), w3.view(torch.uint8), 'ln -> float8 fc codes')
    assert_bit_equal(f3.weight_scale_inv.data, sc3, 'ln -> float8 fc block scales')
    sf.scale_fc_fc(f1, f2, s.to(dev))
    assert_bit_equal(f1.weight.data.view(torch.uint8), w1.view(torch.uint8), 'fc1 float8 codes')
    assert_bit_equal(f1.weight_scale_inv.data, sc1, 'fc1 block scales')
    assert_bit_equal(f2.weight.data.view(torch.uint8), w2.view(torch.uint8), 'fc2 float8 codes')
    assert_bit_equal(f2.weight_scale_inv.data, sc2, 'fc2 block scales')


# ---- Awq.subset_transform: search, fold, rescale the cached inputs (awq.py:299-373) ---------------------------
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_subset_transform_folds_the_found_scales(dev, dtype):
    """A norm in front of two Linears, then a Linear in front of a Linear: the scales are those of the search (the
    oracle evaluated on the device tensors, so both sides see the same GEMMs), the operator in front is divided and
    the Linears multiplied by them with torch's own element-wise results, the cached inputs are divided; subsets the
    reference leaves alone are left alone."""
    from lightcompress_amd.awq import Awq
    K, I, T = 256, 384, 96
    g = gen(91)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    dspec = Q.IntSpec(4, False, 'per_group', group_size=128)
    dspec.qmin, dspec.qmax = dspec.qmin.to(dev), dspec.qmax.to(dev)
    norm = torch.nn.LayerNorm(K).to(dtype)
    norm.weight.data = (torch.rand(K, generator=g) + 0.5).to(dtype)
    norm.bias.data = (torch.randn(K, generator=g) * 0.1).to(dtype)
    gate, up, down = (torch.nn.Linear(K, I, bias=False), torch.nn.Linear(K, I, bias=False), torch.nn.Linear(I, K, bias=False))
    for m in (gate, up, down):
        m.weight.data = torch.randn(m.weight.shape, generator=g) * 0.03
    norm, gate, up, down = (m.to(device=dev, dtype=dtype) for m in (norm, gate, up, down))
    x = (torch.randn(2, T, K, generator=g) * torch.exp(torch.randn(K, generator=g))).to(dtype).to(dev)

    class Mlp(torch.nn.Module):
        def forward(self, xx):
            return down(torch.nn.functional.silu(gate(xx)) * up(xx))
    awq = Awq({'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128), 'special': {}})
    w0 = {'gate': gate.weight.data.clone(), 'up': up.weight.data.clone()}
    nw0, nb0 = norm.weight.data.clone(), norm.bias.data.clone()
    want_scale, _ = A.search_scale(w0, x, lambda xx, ww: down(torch.nn.functional.silu(xx @ ww['gate'].t()) * (xx @ ww['up'].t())), dspec)
    feat = {'gate': [x.clone()], 'up': [x.clone()]}
    awq.subset_transform({'layers': {'gate': gate, 'up': up}, 'prev_op': [norm], 'input': ['gate'], 'inspect': Mlp()}, feat, {})
    assert_bit_equal(norm.weight.data, nw0 / want_scale, 'norm weight / s')
    assert_bit_equal(norm.bias.data, nb0 / want_scale, 'norm bias / s')
    assert_bit_equal(gate.weight.data, w0['gate'] * want_scale.view(1, -1), 'gate * s')
    assert_bit_equal(up.weight.data, w0['up'] * want_scale.view(1, -1), 'up * s')
    assert_bit_equal(feat['gate'][0], x / want_scale.view(1, -1), 'cached input / s')
    assert_bit_equal(feat['up'][0], x / want_scale.view(1, -1), 'cached input / s')
    # a Linear of the same width in front of one Linear (v_proj -> o_proj): rows of the first divided, with its bias
    v, o = torch.nn.Linear(K, K, bias=True), torch.nn.Linear(K, K, bias=False)
    for m in (v, o):
        m.weight.data = torch.randn(m.weight.shape, generator=g) * 0.03
    v, o = v.to(device=dev, dtype=dtype), o.to(device=dev, dtype=dtype)
    vw0, vb0, ow0 = v.weight.data.clone(), v.bias.data.clone(), o.weight.data.clone()
    s2, _ = A.search_scale({'o': ow0}, x, lambda xx, ww: xx @ ww['o'].t(), dspec)
    feat = {'o': [x.clone()]}
    awq.subset_transform({'layers': {'o': o}, 'prev_op': [v], 'input': ['o'], 'inspect': o}, feat, {})
    assert_bit_equal(v.weight.data, vw0 / s2.view(-1, 1), 'v rows / s')
    assert_bit_equal(v.bias.data, vb0 / s2, 'v bias / s')
    assert_bit_equal(o.weight.data, ow0 * s2.view(1, -1), 'o * s')
    assert_bit_equal(feat['o'][0], x / s2.view(1, -1), 'cached input / s')
    # a Linear-like replacement module in front (the reference's _LLMC_LINEAR_TYPES_) is scaled like an nn.Linear
    from lightcompress_amd.module_utils import FakeQuantLinear
    v.weight.data.copy_(vw0); v.bias.data.copy_(vb0); o.weight.data.copy_(ow0)
    fv = FakeQuantLinear.new(v, w_qdq=lambda m: m.weight, a_qdq=None)
    awq.subset_transform({'layers': {'o': o}, 'prev_op': [fv], 'input': ['o'], 'inspect': o}, {'o': [x.clone()]}, {})
    assert_bit_equal(fv.weight.data, vw0 / s2.view(-1, 1), 'replacement module rows / s')
    assert_bit_equal(o.weight.data, ow0 * s2.view(1, -1), 'o * s behind a replacement module')
    # grouped-query attention: v_proj is narrower than o_proj; with do_gqa_trans the statistics come from v_proj's output
    # on the input recorded one entry earlier, and the scales are repeated over the query heads of a group
    heads, kvh, hd = 8, 2, K // 8
    gq = Awq({'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128), 'special': dict(do_gqa_trans=True)})
    gq.set_model_config(types.SimpleNamespace(hidden_size=K, num_attention_heads=heads, num_key_value_heads=kvh))
    vk, og = torch.nn.Linear(K, kvh * hd, bias=False), torch.nn.Linear(K, K, bias=False)
    for m in (vk, og):
        m.weight.data = torch.randn(m.weight.shape, generator=g) * 0.03
    vk, og = vk.to(device=dev, dtype=dtype), og.to(device=dev, dtype=dtype)
    vw0, ow0 = vk.weight.data.clone(), og.weight.data.clone()
    attn = (torch.randn(2, T, K, generator=g)).to(dtype).to(dev)
    s_kv, _ = A.search_scale({'o': ow0}, x, lambda xx, ww: xx @ ww['o'].t(), dspec, gqa=(lambda xx: xx @ vw0.t(), kvh, hd, heads // kvh))
    feat = {'v': [x.clone()], 'o': [attn.clone()]}
    gq.subset_transform({'layers': {'o': og}, 'prev_op': [vk], 'input': ['o'], 'inspect': og}, feat, {})
    rep = A.repeat_gqa(s_kv, kvh, hd, heads // kvh)
    assert_bit_equal(vk.weight.data, vw0 / s_kv.view(-1, 1), 'v rows / s (grouped)')
    assert_bit_equal(og.weight.data, ow0 * rep.view(1, -1), 'o * repeated s')
    assert_bit_equal(feat['o'][0], attn / rep.view(1, -1), 'cached attention output / repeated s')
    assert torch.equal(feat['v'][0], x)
    # left alone: do_trans False, no operator in front, a predecessor of another width without grouped-query scaling
    before = o.weight.data.clone()
    narrow = torch.nn.Linear(K, K // 4, bias=False).to(device=dev, dtype=dtype)
    for sub in ({'do_trans': False, 'prev_op': [v]}, {'prev_op': []}, {'prev_op': [None]}, {'prev_op': [narrow]}):
        awq.subset_transform(dict({'layers': {'o': o}, 'input': ['o'], 'inspect': o}, **sub), {'o': [x.clone()]}, {})
        assert torch.equal(o.weight.data, before)
