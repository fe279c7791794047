"""RTN: the quantizer selection and the deploy-time partials of the reference's base class (rtn.py,
base_blockwise_quantization.py:50-100, 137-257, 348-376, 590-611) against the oracle, bit for bit."""
import pytest
import torch

from oracle import quant_ref as Q
from tests.helpers import assert_bit_equal, gen, weight_like

pytestmark = pytest.mark.gpu


def _linear(w, dev):
    m = torch.nn.Linear(w.shape[1], w.shape[0], bias=False, dtype=w.dtype, device=dev)
    m.weight.data.copy_(w)
    return m


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
def test_rtn_partials_int4_weights_int8_tokens(dev, dtype):
    from lightcompress_amd import FloatQuantizer, IntegerQuantizer
    from lightcompress_amd.rtn import RTN
    cfg = {'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128),
           'act': dict(bit=8, symmetric=True, granularity='per_token')}
    rtn = RTN(cfg)
    assert type(rtn.wquantizer) is IntegerQuantizer and type(rtn.aquantizer) is IntegerQuantizer
    assert rtn.w_only is False and rtn.act_static is False and cfg['weight']['tp'] == 1
    w = weight_like(256, 1024, seed=5, dtype=dtype)
    m = _linear(w, dev)
    wspec, aspec = Q.IntSpec(4, False, 'per_group', group_size=128), Q.IntSpec(8, True, 'per_token')
    params = rtn.get_replacement_params('fake_quant')
    assert_bit_equal(params['w_qdq'](m), Q.int_fake_quant_dynamic(wspec, w), 'w_qdq')
    x = (torch.randn(3, 40, 1024, generator=gen(6)) * 2).to(dtype)
    assert_bit_equal(params['a_qdq'](x.to(dev), m), Q.int_fake_quant_dynamic(aspec, x), 'a_qdq')
    assert rtn.get_replacement_params('fake_quant', w_only=True)['a_qdq'] is None
    real = rtn.get_replacement_params('vllm_quant')
    assert real['quant_config'] is cfg
    for got, want in zip(real['w_q'](m), Q.int_real_quant_dynamic(wspec, w)):
        assert_bit_equal(got, want, 'w_q')
    with pytest.raises(NotImplementedError):
        rtn.get_replacement_params('online_rotate')
    # the qparams the methods that need them up front (GPTQ, static export) find on the layers
    rtn.collect_block_qparams({'fc': m})
    _, os_, oz, oqmax, oqmin = Q.int_tensor_qparams(wspec, w)
    assert_bit_equal(m.buf_scales, os_, 'buf_scales'); assert_bit_equal(m.buf_zeros, oz, 'buf_zeros')
    assert float(m.buf_qmax) == float(oqmax) and float(m.buf_qmin) == float(oqmin)
    assert rtn.subset_transform({'layers': {'fc': m}}, {}, {}) is None
    # float quantizers by configuration
    f = RTN({'weight': dict(quant_type='float-quant', bit='e4m3', symmetric=True, granularity='per_channel', use_qtorch=True)})
    assert type(f.wquantizer) is FloatQuantizer and f.w_only and f.aquantizer is None
    assert_bit_equal(f.w_qdq(m, f.wquantizer), Q.float_fake_quant_dynamic(Q.FloatSpec('e4m3', 'per_channel'), w), 'float w_qdq')


def test_rtn_static_activations_and_clip_factors(dev):
    from lightcompress_amd.rtn import RTN
    cfg = {'weight': dict(bit=8, symmetric=True, granularity='per_channel'),
           'act': dict(bit=8, symmetric=True, granularity='per_tensor', static=True)}
    rtn = RTN(cfg)
    assert rtn.act_static and cfg['act']['calib_algo'] == 'static_minmax'
    w = weight_like(64, 256, seed=7, dtype=torch.bfloat16)
    m = _linear(w, dev)
    acts = [(torch.randn(2, 32, 256, generator=gen(8 + i)) * (1 + i)).bfloat16() for i in range(4)]
    rtn.register_act_qparams({'fc': m, 'norm': torch.nn.LayerNorm(256)}, [a.to(dev) for a in acts])
    spec = Q.IntSpec(8, True, 'per_tensor')
    lo, hi = Q.static_minmax_ranges(spec, list(acts))
    os_, oz, oqmax, oqmin = Q.int_qparams(spec, lo[0], hi[0])
    assert torch.equal(m.buf_act_scales_0.cpu().reshape(-1), os_.reshape(-1))
    x = (torch.randn(5, 256, generator=gen(20)) * 2).bfloat16()
    got = rtn.a_qdq(x.to(dev), m, rtn.aquantizer)
    assert_bit_equal(got, Q.int_fake_quant_static(spec, x, os_, oz, oqmax, oqmin), 'static a_qdq')
    with pytest.raises(AssertionError):
        RTN({'weight': dict(bit=8, symmetric=True, granularity='per_channel'),
             'act': dict(bit=8, symmetric=True, granularity='per_token', static=True)})
    # clip factors registered by the v2 clipper drive the learnable range of w_qdq (quant.py:207-221)
    lc = RTN({'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128, calib_algo='learnable'),
              'special': dict(weight_clip=True, clip_version='v2')})
    assert lc.auto_clipper.clip_version == 'v2'
    up = torch.where(torch.rand(64 * 2, 1, generator=gen(9)) < 0.5, 0.0, 20.0).bfloat16()
    m.register_buffer('buf_upbound_factor', up.to(dev))
    m.register_buffer('buf_lowbound_factor', up.to(dev))
    wspec = Q.IntSpec(4, False, 'per_group', group_size=128)
    rows = Q.reshape_rows(wspec, w)
    rlo, rhi = Q.learnable_range(wspec, rows, lowbound_factor=up, upbound_factor=up)
    s, z, qmax, qmin = Q.int_qparams(wspec, rlo, rhi)
    want = Q.restore_rows(wspec, Q.int_quant_dequant(wspec, rows, s, z, qmax, qmin), w.shape).to(w.dtype)
    assert_bit_equal(lc.w_qdq(m, lc.wquantizer), want, 'w_qdq with clip factors')


def test_rtn_float8_blockwise_weight(dev):
    """A float8 block-wise checkpoint weight: bf16 <- weight * scale_inv, fake quantization, back to float8 with fresh
    block scales (base_blockwise_quantization.py:57-69)."""
    from lightcompress_amd.kernel import weight_cast_to_bf16, weight_cast_to_fp8
    from lightcompress_amd.rtn import RTN
    rtn = RTN({'weight': dict(bit=4, symmetric=True, granularity='per_group', group_size=128)})
    w = weight_like(256, 512, seed=11, dtype=torch.bfloat16).to(dev)
    w8, s8 = weight_cast_to_fp8(w.contiguous())
    m = torch.nn.Module()
    m.weight = torch.nn.Parameter(w8, requires_grad=False)
    m.weight_scale_inv = torch.nn.Parameter(s8.clone(), requires_grad=False)
    back = weight_cast_to_bf16(w8, s8).to(torch.bfloat16)
    want = Q.int_fake_quant_dynamic(Q.IntSpec(4, True, 'per_group', group_size=128), back.cpu())
    want8, wants = weight_cast_to_fp8(want.to(dev).contiguous())
    got = rtn.w_qdq(m, rtn.wquantizer)
    assert got.dtype == torch.float8_e4m3fn
    assert_bit_equal(got.view(torch.uint8), want8.view(torch.uint8), 'float8 codes')
    assert_bit_equal(m.weight_scale_inv.data, wants, 'fresh block scales')


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_fake_quant_modules_apply_the_partials(dev, dtype):
    """FakeQuantLinear / EffcientFakeQuantLinear (module_utils.py:679-858) with the partials of get_replacement_params:
    the forward is the library GEMM of the fake-quantized activations and weight, so with the oracle's tensors moved to
    the device the same torch GEMM gives the same bits."""
    from lightcompress_amd.module_utils import EffcientFakeQuantLinear, FakeQuantLinear
    from lightcompress_amd.rtn import RTN
    cfg = {'weight': dict(bit=4, symmetric=False, granularity='per_group', group_size=128),
           'act': dict(bit=8, symmetric=True, granularity='per_token')}
    rtn = RTN(cfg)
    params = rtn.get_replacement_params('fake_quant')
    w = weight_like(192, 512, seed=31, dtype=dtype)
    m = torch.nn.Linear(512, 192, bias=True, dtype=dtype, device=dev)
    m.weight.data.copy_(w)
    b = m.bias.data.clone()
    m.register_buffer('buf_marker', torch.ones(3, device=dev))
    x = (torch.randn(2, 24, 512, generator=gen(32)) * 2).to(dtype)
    wq = Q.int_fake_quant_dynamic(Q.IntSpec(4, False, 'per_group', group_size=128), w).to(dev)
    xq = Q.int_fake_quant_dynamic(Q.IntSpec(8, True, 'per_token'), x).to(dev)
    want = torch.nn.functional.linear(xq, wq, b)
    for cls in (FakeQuantLinear, EffcientFakeQuantLinear):
        new = cls.new(m, **params)
        assert torch.equal(new.buf_marker, m.buf_marker) and (new.in_features, new.out_features) == (512, 192)
        assert_bit_equal(new(x.to(dev)), want, cls.__name__)
        assert f'weight_quant=w_qdq,act_quant=a_qdq' in repr(new) and repr(new).startswith(cls.__name__ + '(')
    assert_bit_equal(EffcientFakeQuantLinear.new(m, **params).weight, wq, 'quantized once at construction')
    lazy = FakeQuantLinear.new(m, **params)
    assert torch.equal(lazy.weight, m.weight.data) and not hasattr(lazy, 'tmp_weight')
    lazy(x.to(dev))
    assert_bit_equal(lazy.tmp_weight, wq, 'quantized on the first forward')
    lazy.weight.data.mul_(2)                                     # a later change of the weight is seen only on request
    assert_bit_equal(lazy(x.to(dev)), want, 'cached weight')
    lazy.dynamic_quant_weight = True
    assert not torch.equal(lazy(x.to(dev)), want)
    m.weight.data.copy_(w)                                       # (the module's buffer is the layer's own weight tensor)
    # weight only
    wo = FakeQuantLinear.new(m, **rtn.get_replacement_params('fake_quant', w_only=True))
    assert_bit_equal(wo(x.to(dev)), torch.nn.functional.linear(x.to(dev), wq, b), 'weight only')
    assert 'act_quant=None' in repr(wo)
