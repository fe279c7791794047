"""GPU parity of the deploy entry: VllmRealQuantLinear.new / AutoawqRealQuantLinear.new end to end
(module_utils.py:874-927, 1052-1095 of the reference) - w_q -> pack -> buffers with the names vLLM / SGLang /
AutoAWQ load - against the CPU oracle's quantizer and pack restatements."""
import types

import pytest
import torch

from oracle import pack_ref, quant_ref as Q
from tests.helpers import assert_bit_equal, gen, weight_like

pytestmark = pytest.mark.gpu


class Lin(torch.nn.Module):
    def __init__(self, w, bias=None):
        super().__init__()
        self.weight = torch.nn.Parameter(w, requires_grad=False)
        self.bias = None if bias is None else torch.nn.Parameter(bias, requires_grad=False)
        self.out_features, self.in_features = w.shape


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('need_pack', [True, False])
def test_vllm_new_int4_symmetric(dev, dtype, need_pack):
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.module_utils import VllmRealQuantLinear
    R, K = 192, 1024
    w = weight_like(R, K, seed=3, dtype=dtype)
    b = torch.randn(R, generator=gen(4)).to(dtype)
    q = IntegerQuantizer(4, True, 'per_group', group_size=128)
    cfg = {'weight': {'bit': 4, 'symmetric': True, 'granularity': 'per_group', 'group_size': 128, 'need_pack': need_pack}}
    m = Lin(w.to(dev), b.to(dev))
    new = VllmRealQuantLinear.new(m, lambda mod: q.real_quant_weight_dynamic(mod.weight.data), cfg)
    spec = Q.IntSpec(4, True, 'per_group', group_size=128)
    oc, os_, oz = Q.int_real_quant_dynamic(spec, w)
    assert oz is None
    sd = new.state_dict()
    if need_pack:
        op, os16 = pack_ref.pack_ct(oc, os_, 4)
        assert set(sd) == {'weight_packed', 'bias', 'weight_scale'}
        assert_bit_equal(sd['weight_packed'], op, 'weight_packed')
        assert_bit_equal(sd['weight_scale'], os16, 'weight_scale')
        assert torch.equal(pack_ref.unpack_ct(sd['weight_packed'].cpu(), 4, K), oc)
        assert new.weight_shape == (R, K // 8) and new.weight_dtype == torch.int32 and new.scales_dtype == torch.float16
    else:
        assert set(sd) == {'weight', 'bias', 'weight_scale'}
        assert_bit_equal(sd['weight'], oc, 'weight')
        assert_bit_equal(sd['weight_scale'], os_, 'weight_scale')
    assert new.input_scale is None and new.zeros_shape is None and new.zeros_dtype is None
    assert_bit_equal(sd['bias'], b, 'bias')
    assert (new.in_features, new.out_features) == (K, R) and new.scales_shape == (R, K // 128)
    with pytest.raises(NotImplementedError):
        new(torch.zeros(1, K, device=dev))
    # the SGLang module (module_utils.py:1010-1026) is the same container under its own name
    from lightcompress_amd.module_utils import SglRealQuantLinear
    sgl = SglRealQuantLinear.new(Lin(w.to(dev), b.to(dev)), lambda mod: q.real_quant_weight_dynamic(mod.weight.data), cfg)
    assert type(sgl) is SglRealQuantLinear and set(sgl.state_dict()) == set(sd)
    for k in sd:
        assert torch.equal(sgl.state_dict()[k], sd[k])
    assert repr(sgl).startswith(f'SglRealQuantLinear(in_features={K}, out_features={R}, bias=True, weight_shape=')
    assert repr(new).startswith('VllmRealQuantLinear(') and 'zeros_dtype=None' in repr(new)


def test_vllm_new_int8_static_activation_scale(dev):
    """w8a8 static: int8 codes stay unpacked, buf_act_scales_0 becomes input_scale with a leading axis (module_utils.py:880-888)."""
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.module_utils import VllmRealQuantLinear
    R, K = 96, 512
    w = weight_like(R, K, seed=5, dtype=torch.bfloat16)
    q = IntegerQuantizer(8, True, 'per_channel')
    cfg = {'weight': {'bit': 8, 'symmetric': True, 'granularity': 'per_channel'},
           'act': {'bit': 8, 'symmetric': True, 'granularity': 'per_tensor', 'static': True}}
    m = Lin(w.to(dev))
    m.buf_act_scales_0 = torch.tensor(0.0123, device=dev)
    new = VllmRealQuantLinear.new(m, lambda mod: q.real_quant_weight_dynamic(mod.weight.data), cfg)
    oc, os_, _ = Q.int_real_quant_dynamic(Q.IntSpec(8, True, 'per_channel'), w)
    assert_bit_equal(new.weight, oc, 'int8 weight')
    assert new.weight.dtype == torch.int8 and new.bias is None
    assert_bit_equal(new.weight_scale, os_, 'weight_scale')
    assert new.input_scale.shape == (1,) and float(new.input_scale) == pytest.approx(0.0123)
    assert set(new.state_dict()) == {'weight', 'weight_scale', 'input_scale'}


def test_vllm_new_fp8_from_blockwise_checkpoint(dev):
    """The module holds a block-wise float8 weight (weight_scale_inv, block_size): quant_pack first brings it back to
    bf16 (module_utils.py:915-921), then FP8 per-channel real quantization; per_block targets name their scales
    weight_scale_inv (:897-900)."""
    from lightcompress_amd import FloatQuantizer
    from lightcompress_amd.module_utils import VllmRealQuantLinear
    R, K = 256, 384
    w = weight_like(R, K, seed=6, dtype=torch.bfloat16, std=0.006, outlier_frac=0.0005, outlier_mul=30)
    y, sc = Q.triton_weight_cast_to_fp8(w)
    wb = Q.triton_weight_cast_to_bf16(y, sc).to(torch.bfloat16)
    m = Lin(y.to(dev))
    m.weight_scale_inv = torch.nn.Parameter(sc.to(dev), requires_grad=False)
    m.block_size = 128
    q = FloatQuantizer('e4m3', True, 'per_channel', use_qtorch=True)
    cfg = {'weight': {'bit': 'e4m3', 'symmetric': True, 'granularity': 'per_channel'}, 'quant_type': 'float-quant'}
    new = VllmRealQuantLinear.new(m, lambda mod: q.real_quant_weight_dynamic(mod.weight.data), cfg)
    assert m.weight.data.dtype == torch.bfloat16
    assert_bit_equal(m.weight.data, wb, 'bf16 weight restored from the block-wise float8 checkpoint')
    oc, os_, _ = Q.float_real_quant_dynamic(Q.FloatSpec('e4m3', 'per_channel'), wb)
    assert_bit_equal(new.weight.view(torch.uint8), oc.view(torch.uint8), 'float8 codes')
    assert_bit_equal(new.weight_scale, os_, 'weight_scale')
    # a per_block target: scales are registered as weight_scale_inv
    qb = FloatQuantizer('e4m3', True, 'per_block', block_size=128, use_qtorch=True)
    cfgb = {'weight': {'bit': 'e4m3', 'symmetric': True, 'granularity': 'per_block', 'block_size': 128}}
    m2 = Lin(wb.to(dev))
    new2 = VllmRealQuantLinear.new(m2, lambda mod: qb.real_quant_weight_dynamic(mod.weight.data), cfgb)
    oy, osc, _ = Q.float_per_block_real_quant(Q.FloatSpec('e4m3', 'per_block'), wb)
    assert set(new2.state_dict()) == {'weight', 'weight_scale_inv'}
    assert_bit_equal(new2.weight.view(torch.uint8), oy.view(torch.uint8), 'per_block codes')
    assert_bit_equal(new2.weight_scale_inv, osc, 'per_block scales')


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_autoawq_new(dev, dtype):
    from lightcompress_amd import IntegerQuantizer
    from lightcompress_amd.module_utils import AutoawqRealQuantLinear
    R, K = 320, 1024
    w = weight_like(R, K, seed=8, dtype=dtype)
    b = torch.randn(R, generator=gen(9)).to(dtype)
    spec = Q.IntSpec(4, False, 'per_group', group_size=128)
    q = IntegerQuantizer(4, False, 'per_group', group_size=128)
    cfg = {'weight': {'bit': 4, 'symmetric': False, 'granularity': 'per_group', 'group_size': 128, 'pack_version': 'gemm_pack'}}
    m = Lin(w.to(dev), b.to(dev))
    # fp16 rows are quantized in fp32 by the GPU quantizer; the reference's w_q hands scales in the weight dtype
    def w_q(mod):
        wt = mod.weight.data
        c, s, z = q.real_quant_weight_dynamic(wt.float() if wt.dtype == torch.float16 else wt)
        return c, s.to(wt.dtype), z
    new = AutoawqRealQuantLinear.new(m, w_q, cfg)
    _, os_, oz = Q.int_real_quant_dynamic(spec, w.float() if dtype == torch.float16 else w)
    want = pack_ref.gemm_pack(w, os_.to(dtype), oz, 128)
    sd = new.state_dict()
    assert set(sd) == {'qweight', 'bias', 'scales', 'qzeros'}
    for name, t in zip(('qweight', 'scales', 'qzeros'), want):
        assert_bit_equal(sd[name], t, name)
    assert new.weight_shape == (K, R // 8) and new.scales_shape == (K // 128, R) and new.zeros_shape == (K // 128, R // 8)
    assert new.weight_dtype == torch.int32 and new.scales_dtype == torch.float16 and new.zeros_dtype == torch.int32
    # the packed integers are the quantizer's codes
    oc, _, _ = Q.int_real_quant_dynamic(spec, w.float() if dtype == torch.float16 else w)
    iw = pack_ref.gemm_unpack(sd['qweight'].cpu())
    assert float((iw.t() == oc).float().mean()) > 0.99           # gemm_pack re-rounds (w + z s) / s with the scales cast to fp16
    cfg['weight']['pack_version'] = 'gemv_pack'
    with pytest.raises(NotImplementedError):
        AutoawqRealQuantLinear.new(Lin(w.to(dev)), w_q, cfg)
