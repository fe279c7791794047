"""Scale folding of the block-wise algorithms with the reference's method names, running on liblcq.

Mirrors the members of ``BaseBlockwiseQuantization`` (llmc/compression/quantization/
base_blockwise_quantization.py of ModelTC/LightCompress) that AWQ-style methods call after a scale search:
``apply_scale`` (:619-636), ``scale_fc_fc`` (:664-723), ``scale_ln_fcs`` (:772-801), ``repeat_gqa_scales``
(:613-617), ``scaling_input`` (:899-912) and ``update_input_feat`` (:914-920).  Use it as a mix-in in front of
the reference's class, or stand-alone.

Float8 block-wise checkpoints (``weight_scale_inv``) go through the block-wise casts of ``kernel.py``: cast to bf16,
scale, cast back, like the reference (:690-699, 711-720).
"""
from __future__ import annotations

import torch

from . import _lib as L

_MUL_COLS, _DIV_COLS, _MUL_ROWS, _DIV_ROWS = 0, 1, 2, 3


def is_linear_like(m):
    """nn.Linear or a module that stands in for one (the reference's _LLMC_LINEAR_TYPES_ / _TRANSFORMERS_LINEAR_TYPES_):
    in_features, out_features and a 2-D weight."""
    if isinstance(m, torch.nn.Linear):
        return True
    w = getattr(m, 'weight', None)
    return hasattr(m, 'in_features') and hasattr(m, 'out_features') and torch.is_tensor(w) and w.dim() == 2


def _scale_(t, s, mode):
    """In place: t (* or /) s along columns (mode 0 / 1) or rows (2 / 3); t [T, K] or [K]."""
    x = t.data
    if not x.is_contiguous():
        raise L.LcqError('in-place scaling needs a contiguous tensor')
    x2 = x.view(1, -1) if x.dim() == 1 else x.view(-1, x.shape[-1])
    s = s.to(device=x.device, dtype=x.dtype).contiguous().view(-1)
    assert s.numel() == (x2.shape[1] if mode < 2 else x2.shape[0])
    L.check(L.lib().lcq_scale_matrix(L.ptr(x2), L.i32(L.dtype_code(x.dtype)), L.i64(x2.shape[0]), L.i64(x2.shape[1]),
                                     L.ptr(s), L.i32(mode), L.ptr(x2), L.stream()), 'lcq_scale_matrix')
    return t


def _scale_fp8_(fc, scales, mode, block_size):
    """A float8 block-wise weight: bf16 <- weight * weight_scale_inv, scale, back to float8 with fresh block scales."""
    from .kernel import weight_cast_to_bf16, weight_cast_to_fp8
    tmp = weight_cast_to_bf16(fc.weight.data, fc.weight_scale_inv, block_size).to(torch.bfloat16)
    _scale_(tmp, scales, mode)
    fc.weight.data, fc.weight_scale_inv.data = weight_cast_to_fp8(tmp, block_size)


class ScaleFolding:
    """Expects, where GQA is used, ``num_key_value_heads``, ``head_dim``, ``num_key_value_groups``, ``has_gqa`` and
    ``do_gqa_trans`` on ``self`` like the reference's class; for fused QKV linears ``model.get_num_attention_heads()``
    or ``num_heads``; for float8 checkpoints ``fp8_block_size``."""

    has_gqa = False
    do_gqa_trans = False
    fp8_block_size = 128

    @torch.no_grad()
    def repeat_gqa_scales(self, scales):
        scales = scales.view(1, self.num_key_value_heads, self.head_dim)
        return torch.repeat_interleave(scales, dim=1, repeats=self.num_key_value_groups)

    @torch.no_grad()
    def apply_scale(self, scales, prev_op, layers):
        assert len(prev_op) == 1, 'Only support single prev_op. If multi prev_ops, code need to be updated.'
        op = prev_op[0]
        if is_linear_like(op):
            assert len(layers) == 1
            self.scale_fc_fc(prev_op[0], layers[0], scales)
        elif hasattr(prev_op[0], 'weight') and prev_op[0].weight.dim() == 1:          # LayerNorm / RMSNorm
            self.scale_ln_fcs(prev_op[0], layers, scales)
        else:
            raise NotImplementedError(f'prev_op {type(prev_op[0])} not supported yet!')

    @torch.no_grad()
    def scale_fc_fc(self, fc1, fc2, scales):
        scales = scales.to(fc1.weight.device)
        has_bias = getattr(fc1, 'bias', None) is not None
        if fc1.out_features == fc2.in_features * 3:
            # fused QKV laid out [head][q, k, v][head_dim] along the output channels (:648-676): only the value rows
            # are divided, row (h, 2, d) by scales[h * head_dim + d]; per head they are one contiguous block
            model = getattr(self, 'model', None)
            num_heads = model.get_num_attention_heads() if model is not None else self.num_heads
            w = fc1.weight.data
            hd = w.shape[0] // (3 * num_heads)
            blocks = w.view(num_heads, 3, hd, w.shape[1])
            sv = scales.view(num_heads, hd)
            for h in range(num_heads):
                _scale_(blocks[h, 2], sv[h], _DIV_ROWS)
            if has_bias:
                b = fc1.bias.data.view(num_heads, 3, hd)
                for h in range(num_heads):
                    _scale_(b[h, 2], sv[h], _DIV_COLS)
        elif fc1.out_features == fc2.in_features * 2:
            half = fc1.weight.data.shape[0] // 2
            _scale_(fc1.weight.data[half:], scales, _DIV_ROWS)
            if has_bias:
                _scale_(fc1.bias.data[half:], scales, _DIV_COLS)
        elif fc1.out_features == fc2.in_features:
            if has_bias:
                _scale_(fc1.bias, scales, _DIV_COLS)
            if fc1.weight.data.dtype == torch.float8_e4m3fn:
                _scale_fp8_(fc1, scales, _DIV_ROWS, self.fp8_block_size)
            else:
                _scale_(fc1.weight, scales, _DIV_ROWS)
        elif self.has_gqa and self.do_gqa_trans:
            if has_bias:
                _scale_(fc1.bias, scales, _DIV_COLS)
            _scale_(fc1.weight, scales, _DIV_ROWS)
            if fc1.out_features != fc2.in_features:
                scales = self.repeat_gqa_scales(scales)
        else:
            raise Exception('Can not scale this fc-fc.')
        if fc2.weight.data.dtype == torch.float8_e4m3fn:
            _scale_fp8_(fc2, scales, _MUL_COLS, self.fp8_block_size)
        else:
            _scale_(fc2.weight, scales, _MUL_COLS)

    @torch.no_grad()
    def scale_ln_fcs(self, ln, fcs, scales):
        if not isinstance(fcs, list):
            fcs = [fcs]
        scales = scales.to(ln.weight.device).to(ln.weight.dtype)
        _scale_(ln.weight, scales, _DIV_COLS)
        if getattr(ln, 'bias', None) is not None:
            _scale_(ln.bias, scales, _DIV_COLS)
        for fc in fcs:
            if fc.weight.data.dtype == torch.float8_e4m3fn:
                _scale_fp8_(fc, scales, _MUL_COLS, self.fp8_block_size)
            else:
                _scale_(fc.weight, scales, _MUL_COLS)
        for p in ln.parameters():
            assert torch.isnan(p).sum() == 0
        for fc in fcs:
            for p in fc.parameters():
                assert torch.isnan(p.float() if p.dtype == torch.float8_e4m3fn else p).sum() == 0

    @torch.no_grad()
    def scaling_input(self, x, scales, is_gqa):
        scales_tmp = self.repeat_gqa_scales(scales) if is_gqa else scales
        x2 = x.contiguous()
        out = torch.empty_like(x2)
        K = x2.shape[-1]
        s = scales_tmp.to(device=x2.device, dtype=x2.dtype).contiguous().view(-1)
        L.check(L.lib().lcq_scale_matrix(L.ptr(x2), L.i32(L.dtype_code(x2.dtype)), L.i64(x2.numel() // K), L.i64(K),
                                         L.ptr(s), L.i32(_DIV_COLS), L.ptr(out), L.stream()), 'lcq_scale_matrix')
        return out

    @torch.no_grad()
    def update_input_feat(self, scale, input_feat, layers_dict, is_gqa):
        for layer_name in layers_dict:
            for i in range(len(input_feat[layer_name])):
                inp = input_feat[layer_name][i]
                scale = scale.to(inp.device)
                input_feat[layer_name][i] = self.scaling_input(inp, scale, is_gqa)
