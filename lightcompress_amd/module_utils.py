"""Real-quantized Linear containers and their packing, with the reference's class API.

Mirrors ``VllmRealQuantLinear`` (module_utils.py:855-955: buffers ``weight`` / ``weight_packed``,
``weight_scale`` / ``weight_scale_inv``, ``input_scale``, ``bias``; ``new``, ``quant_pack``, ``pack``) and
``AutoawqRealQuantLinear`` (module_utils.py:1029-1158: buffers ``qweight``, ``scales``, ``qzeros``, ``bias``;
``new``, ``quant_pack``, ``gemm_pack``) of ModelTC/LightCompress, so that what they hold loads in vLLM / SGLang
(compressed-tensors) and AutoAWQ.  The reference packs on the host (numpy round trip / Python loops over
columns); here both layouts are one kernel over device memory.  ``FakeQuantLinear`` and ``EffcientFakeQuantLinear``
(module_utils.py:679-858) are the modules that apply the ``w_qdq`` / ``a_qdq`` partials in a forward pass.
"""
from __future__ import annotations

import math
from functools import partial

import torch

from . import _lib as L

_CODE = {torch.int32: L.CODE_I32, torch.int8: L.CODE_I8, torch.uint8: L.CODE_U8}


def _bf16_weight(module):
    """module_utils.py:916-921 / 1085-1090: a block-wise float8 checkpoint weight is brought back to bf16 first."""
    if module.weight.data.dtype == torch.float8_e4m3fn:
        from .quant import weight_cast_to_bf16
        module.weight.data = weight_cast_to_bf16(module.weight.data, module.weight_scale_inv.data,
                                                 module.block_size).to(torch.bfloat16)


def _func_name(fn):
    return fn.func.__name__ if isinstance(fn, partial) else fn.__name__


class _FakeQuantBase(torch.nn.Module):
    """What the two fake-quant modules share (module_utils.py:679-710, 775-800): the layer's weight and bias as
    buffers, the `buf_*` entries of the original layer (qparams, clip factors, act-order indices) carried over.
    Online rotation and the block-wise float8 GEMM of float8 checkpoints belong to other paths of the reference and
    raise here."""

    def _adopt(self, weight, bias, ori_module):
        self.register_buffer('weight', weight)
        if bias is not None:
            self.register_buffer('bias', bias)
        else:
            self.bias = None
        for name, buf in list(ori_module.named_buffers()) + list(ori_module.named_parameters()):
            if name.startswith('buf_'):
                self.register_buffer(name, buf.data)
        if getattr(self, 'buf_rotate', False):
            raise NotImplementedError('online rotation is not part of this path')
        self.buf_rotate = False
        if weight.dtype == torch.float8_e4m3fn:
            raise NotImplementedError('forward on block-wise float8 weights (the reference\'s float8 GEMM) is not part of this path')
        self.fp8_forward = False

    @classmethod
    def get_func_name(cls, any_callable):
        return _func_name(any_callable)

    def _name(self, module, w_qdq, a_qdq):
        self.in_features, self.out_features = module.in_features, module.out_features
        self.w_qdq_name = self.get_func_name(w_qdq)
        self.a_qdq_name = self.get_func_name(a_qdq) if a_qdq is not None else 'None'


class FakeQuantLinear(_FakeQuantBase):
    """module_utils.py:679-772: activations through `a_qdq(x, self)`, the weight through `w_qdq(self)` on the first
    forward (kept as `tmp_weight`; again on every forward with `dynamic_quant_weight` / `dynamic_quant_tmp_weight`),
    then the library GEMM."""

    def __init__(self, weight, bias, ori_module, w_qdq, a_qdq):
        super().__init__()
        self._adopt(weight, bias, ori_module)
        self.a_qdq = a_qdq
        self.w_qdq = w_qdq
        self.dynamic_quant_weight = False
        self.dynamic_quant_tmp_weight = False

    def forward(self, x):
        if self.a_qdq is not None:
            x = self.a_qdq(x, self)
        if not hasattr(self, 'tmp_weight'):
            self.register_buffer('tmp_weight', self.w_qdq(self), persistent=False)
            self.tmp_bias = self.bias
        elif self.dynamic_quant_weight:
            self.tmp_weight = self.w_qdq(self)
            self.tmp_bias = self.bias
        elif self.dynamic_quant_tmp_weight:
            self.tmp_weight = self.w_qdq(self)
        return torch.nn.functional.linear(x, self.tmp_weight, self.tmp_bias)

    @classmethod
    @torch.no_grad()
    def new(cls, module, w_qdq, a_qdq):
        bias = module.bias.data if getattr(module, 'bias', None) is not None else None
        new_module = cls(module.weight.data, bias, ori_module=module, w_qdq=w_qdq, a_qdq=a_qdq)
        new_module._name(module, w_qdq, a_qdq)
        return new_module

    def __repr__(self):
        return (f'FakeQuantLinear(in_features={self.in_features},out_features={self.out_features}, '
                f'bias={self.bias is not None},weight_quant={self.w_qdq_name},act_quant={self.a_qdq_name},'
                f'online_rotate={self.buf_rotate})')


class EffcientFakeQuantLinear(_FakeQuantBase):
    """module_utils.py:775-858: the weight is fake-quantized once, when the module is made."""

    def __init__(self, weight, bias, ori_module, a_qdq):
        super().__init__()
        self._adopt(weight, bias, ori_module)
        self.a_qdq = a_qdq

    @torch.no_grad()
    def forward(self, x):
        if self.a_qdq is not None:
            x = self.a_qdq(x, self)
        return torch.nn.functional.linear(x, self.weight, self.bias)

    @classmethod
    @torch.no_grad()
    def new(cls, module, w_qdq, a_qdq, debug_print={}):
        weight = w_qdq(module)
        bias = module.bias.data if module.bias is not None else None
        new_module = cls(weight, bias, ori_module=module, a_qdq=a_qdq)
        new_module._name(module, w_qdq, a_qdq)
        new_module.debug_print = debug_print
        return new_module

    def __repr__(self):
        return (f'EffcientFakeQuantLinear(in_features={self.in_features},out_features={self.out_features},'
                f'bias={self.bias is not None},weight_quant={self.w_qdq_name},act_quant={self.a_qdq_name},'
                f'online_rotate={self.buf_rotate},fp8_forward={self.fp8_forward},debug_print={self.debug_print})')


class _RealQuantLinear(torch.nn.Module):
    @torch.no_grad()
    def forward(self, x):
        raise NotImplementedError

    def _describe(self, module, weight, scales, zeros):
        self.in_features = module.in_features
        self.out_features = module.out_features
        self.weight_shape, self.weight_dtype = weight.shape, weight.dtype
        self.scales_shape, self.scales_dtype = scales.shape, scales.dtype
        self.zeros_shape = zeros.shape if zeros is not None else None
        self.zeros_dtype = zeros.dtype if zeros is not None else None

    def _reg(self, name, value):
        if value is not None:
            self.register_buffer(name, value)
        else:
            setattr(self, name, None)

    def __repr__(self):
        """The one-line description the reference prints for its deploy modules (module_utils.py:995-1008)."""
        fields = ('in_features', 'out_features')
        described = ('weight_shape', 'weight_dtype', 'scales_shape', 'scales_dtype', 'zeros_shape', 'zeros_dtype')
        parts = [f'{k}={getattr(self, k, None)}' for k in fields] + [f'bias={self.bias is not None}']
        parts += [f'{k}={getattr(self, k, None)}' for k in described]
        return f'{type(self).__name__}(' + ', '.join(parts) + ')'


class VllmRealQuantLinear(_RealQuantLinear):
    def __init__(self, weight, bias, scales, input_scale, need_pack, scales_name):
        super().__init__()
        self.register_buffer('weight_packed' if need_pack else 'weight', weight)
        self._reg('bias', bias)
        self.register_buffer(scales_name, scales)
        self.register_buffer('input_scale', input_scale)

    @classmethod
    @torch.no_grad()
    def new(cls, module, w_q, quant_config):
        """module_utils.py:875-911."""
        weight, scales = cls.quant_pack(module, w_q, quant_config)
        input_scale = module.buf_act_scales_0 if hasattr(module, 'buf_act_scales_0') else None
        act = quant_config['act'] if 'act' in quant_config else None
        if act is not None and act.get('static', False) and quant_config.get('quant_type', 'int-quant') == 'int-quant':
            input_scale = input_scale.unsqueeze(0)
        bias = module.bias.data if module.bias is not None else None
        need_pack = quant_config['weight'].get('need_pack', False)
        scales_name = 'weight_scale_inv' if quant_config['weight']['granularity'] == 'per_block' else 'weight_scale'
        new_module = cls(weight, bias, scales, input_scale, need_pack, scales_name)
        new_module._describe(module, weight, scales, None)
        return new_module

    @classmethod
    @torch.no_grad()
    def quant_pack(cls, module, w_q, quant_config):
        """module_utils.py:913-927: w_q(module) -> (codes, scales, zeros), packed when need_pack."""
        _bf16_weight(module)
        weight, scales, zeros = w_q(module)
        if quant_config['weight'].get('need_pack', False):
            weight, scales = cls.pack(weight, scales, quant_config)
        return weight, scales

    @classmethod
    @torch.no_grad()
    def pack(cls, weight, scales, quant_config):
        """-> (int32 [R, ceil(K / (32/bits))], fp16 scales)."""
        num_bits = quant_config['weight']['bit']
        if weight.dtype not in _CODE:
            raise L.LcqError(f'codes must be int32/int8/uint8, got {weight.dtype}')
        w = weight.contiguous()
        R, K = w.shape
        pack_factor = 32 // num_bits
        packed = torch.empty((R, math.ceil(K / pack_factor)), dtype=torch.int32, device=w.device)
        L.check(L.lib().lcq_pack_ct(L.ptr(w), L.i32(_CODE[w.dtype]), L.i64(R), L.i64(K), L.i32(num_bits),
                                    L.ptr(packed), L.stream()), 'lcq_pack_ct')
        return packed, scales.to(torch.float16)

    @classmethod
    @torch.no_grad()
    def quant_pack_fused(cls, weight, wquantizer, quant_config):
        """pack(*wquantizer.real_quant_weight_dynamic(weight)[:2], quant_config) in one kernel: the bf16 / fp32
        weight is read once and only the packed words and the scales are written."""
        assert quant_config['weight']['bit'] == 4
        packed, scales, _ = wquantizer.real_quant_pack_dynamic(weight)
        return packed, scales.to(torch.float16)


class SglRealQuantLinear(VllmRealQuantLinear):
    """module_utils.py:1010-1026: the same buffers and packing under SGLang's name."""


class AutoawqRealQuantLinear(_RealQuantLinear):
    def __init__(self, weight, bias, scales, zeros):
        super().__init__()
        self.register_buffer('qweight', weight)
        self._reg('bias', bias)
        self.register_buffer('scales', scales)
        self._reg('qzeros', zeros)

    @classmethod
    @torch.no_grad()
    def new(cls, module, w_q, quant_config):
        """module_utils.py:1053-1078."""
        weight, scales, zeros = cls.quant_pack(module, w_q, quant_config)
        bias = module.bias.data if module.bias is not None else None
        new_module = cls(weight, bias, scales, zeros)
        new_module._describe(module, weight, scales, zeros)
        return new_module

    @classmethod
    @torch.no_grad()
    def quant_pack(cls, module, w_q, quant_config):
        """module_utils.py:1080-1095."""
        _bf16_weight(module)
        _, scales, zeros = w_q(module)
        pack_version = quant_config['weight']['pack_version']
        if pack_version != 'gemm_pack':
            raise NotImplementedError(f'Not support {pack_version}.')
        return cls.gemm_pack(module, module.weight.data, scales, zeros, quant_config)

    @classmethod
    @torch.no_grad()
    def gemm_pack(cls, module, weight, scales, zeros, quant_config):
        """-> (qweight [K, R/8] int32, scales [K/g, R] fp16, qzeros [K/g, R/8] int32)."""
        assert scales is not None and zeros is not None
        bit = quant_config['weight']['bit']
        if bit != 4:
            raise NotImplementedError('Only 4-bit are supported for now.')
        group_size = quant_config['weight']['group_size']
        w = weight.data.contiguous()
        R, K = w.shape
        if module is not None:
            assert module.in_features == K
        s = scales.to(w.dtype).contiguous()
        z = zeros.to(torch.int32).contiguous()
        G = K // group_size
        qweight = torch.empty((K, R // 8), dtype=torch.int32, device=w.device)
        s16 = torch.empty((G, R), dtype=torch.float16, device=w.device)
        qzeros = torch.empty((G, R // 8), dtype=torch.int32, device=w.device)
        L.check(L.lib().lcq_pack_awq(L.ptr(w), L.i32(L.dtype_code(w.dtype)), L.ptr(s), L.ptr(z), L.i64(R), L.i64(K),
                                     L.i32(group_size), L.ptr(qweight), L.ptr(s16), L.ptr(qzeros), L.stream()),
                'lcq_pack_awq')
        return qweight, s16, qzeros
