"""Packing of real-quantized weights with the reference's classmethod API.

Mirrors ``VllmRealQuantLinear.pack`` (module_utils.py:929-955) and
``AutoawqRealQuantLinear.gemm_pack`` (module_utils.py:1097-1158) of
ModelTC/LightCompress.  The reference packs on the host (numpy round trip /
Python loops over columns); here both layouts are one kernel over device
memory.  The nn.Module containers around them are not part of this path.
"""
from __future__ import annotations

import math

import torch

from . import _lib as L

_CODE = {torch.int32: L.CODE_I32, torch.int8: L.CODE_I8, torch.uint8: L.CODE_U8}


class VllmRealQuantLinear:
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
    def quant_pack(cls, weight, wquantizer, quant_config):
        """pack(*wquantizer.real_quant_weight_dynamic(weight)[:2], quant_config) in one kernel: the bf16 / fp32
        weight is read once and only the packed words and the scales are written."""
        assert quant_config['weight']['bit'] == 4
        packed, scales, _ = wquantizer.real_quant_pack_dynamic(weight)
        return packed, scales.to(torch.float16)


class AutoawqRealQuantLinear:
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
