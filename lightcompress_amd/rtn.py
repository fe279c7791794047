"""Round-to-nearest: the quantizer selection and the per-layer partials every block-wise method of the reference
inherits, on liblcq.

``rtn.py`` of ModelTC/LightCompress adds nothing to ``BaseBlockwiseQuantization`` (its ``subset_transform`` is empty):
round-to-nearest IS the base class' deploy-time partials - ``w_qdq`` (fake quantization of a layer's weight,
base_blockwise_quantization.py:50-71), ``w_q`` (real quantization, :73-74), ``a_qdq`` (activations, dynamic or with the
registered static qparams, :76-86) - over the quantizers that ``set_quant_config`` picks from the configuration
(:154-207, 233-251).  ``RTN`` here is those members with the reference's names; the model walk around them (blocks,
hooks, module replacement) stays the reference's.
"""
from __future__ import annotations

from functools import partial

import torch

from .auto_clip import AutoClipper
from .blockwise import ScaleFolding, is_linear_like
from .kernel import weight_cast_to_bf16, weight_cast_to_fp8
from .quant import FloatQuantizer, IntegerQuantizer, Weight48IntegerQuantizer

_REALQUANT_MODES = ('vllm_quant', 'sgl_quant', 'autoawq_quant')


def select_quantizer(cfg):
    """base_blockwise_quantization.py:156-165, 174-181: the quantizer class a `weight` / `act` section asks for."""
    quant_type = cfg.get('quant_type', 'int-quant')
    if quant_type == 'int-quant':
        return Weight48IntegerQuantizer if cfg['bit'] == 48 else IntegerQuantizer
    if quant_type == 'float-quant':
        return FloatQuantizer
    raise ValueError(f'quant_type: {quant_type}')


class RTN(ScaleFolding):
    def __init__(self, quant_config, padding_mask=None, fp8_block_size=128):
        self.quant_config = quant_config
        self.padding_mask = padding_mask
        self.fp8_block_size = fp8_block_size
        self.set_quant_config()

    def set_quant_config(self):
        """The part of base_blockwise_quantization.py:137-257 that concerns the quantizers of the path."""
        qc = self.quant_config
        self.quant_out = qc.get('quant_out', False)
        self.tp = qc.get('tp', 1)
        qc['weight']['tp'] = self.tp
        self.weight_quant_module = select_quantizer(qc['weight'])
        self.wquantizer = self.weight_quant_module(**qc['weight'])
        if 'act' in qc:
            if qc['weight']['granularity'] == 'per_block':
                assert qc['act']['granularity'] == 'per_group'
                assert qc['act']['group_size'] == qc['weight']['block_size']
            self.w_only = False
            self.act_quant_module = select_quantizer(qc['act'])
            self.act_static = qc['act'].get('static', False)
            if self.act_static:
                assert qc['act']['granularity'] == 'per_tensor', 'Only support per_tensor static quant'
                if qc['act'].get('calib_algo', 'minmax') == 'minmax':
                    qc['act']['calib_algo'] = 'static_minmax'
            qc['act']['tp'] = self.tp
            self.aquantizer = self.act_quant_module(**qc['act'])
        else:
            self.w_only = True
            self.aquantizer = None
            self.act_static = False
        special_config = qc.get('special', {})
        self.true_sequential = special_config.get('true_sequential', False)
        self.weight_clip = special_config.get('weight_clip', False)
        if self.weight_clip or special_config.get('search_clip_init', False):
            self.save_clip = special_config.get('save_clip', False)
            self.clip_version = special_config.get('clip_version', 'v1')
            if self.clip_version == 'v2':
                assert self.wquantizer.calib_algo == 'learnable'
            clip_sym = special_config.get('clip_sym', self.wquantizer.sym)
            self.auto_clipper = AutoClipper(w_only=self.w_only, wquantizer=self.wquantizer, aquantizer=self.aquantizer,
                                            clip_version=self.clip_version, clip_sym=clip_sym, save_clip=self.save_clip,
                                            padding_mask=self.padding_mask)

    # -- the partials handed to the replacement modules -------------------------------------------------------
    @torch.no_grad()
    def w_qdq(self, module, wquantizer):
        """Fake quantization of a layer's weight with the clip factors it carries, if any; a float8 block-wise weight
        goes through bf16 and comes back as float8 with fresh block scales."""
        args = {'lowbound_factor': getattr(module, 'buf_lowbound_factor', None),
                'upbound_factor': getattr(module, 'buf_upbound_factor', None)}
        is_fp8 = module.weight.data.dtype == torch.float8_e4m3fn
        if is_fp8:
            weight = weight_cast_to_bf16(module.weight, module.weight_scale_inv, self.fp8_block_size).to(torch.bfloat16)
        else:
            weight = module.weight
        weight = wquantizer.fake_quant_weight_dynamic(weight, args)
        if is_fp8:
            weight, module.weight_scale_inv.data = weight_cast_to_fp8(weight, self.fp8_block_size)
        return weight

    @torch.no_grad()
    def w_q(self, module, wquantizer):
        return wquantizer.real_quant_weight_dynamic(module.weight.data)

    @torch.no_grad()
    def a_qdq(self, act, module, aquantizer, input_index=0):
        if self.act_static:
            args = {k: getattr(module, f'buf_act_{k}_{input_index}', None) for k in ('scales', 'zeros', 'qmax', 'qmin')}
            return aquantizer.fake_quant_act_static(act, args)
        return aquantizer.fake_quant_act_dynamic(act)

    def get_replacement_params(self, mode='fake_quant', w_only=False, name=None):
        """base_blockwise_quantization.py:88-100 for the modes of this path."""
        if mode in ('fake_quant', 'fake_quant_wo_kv'):
            return {'a_qdq': None if w_only else partial(self.a_qdq, aquantizer=self.aquantizer),
                    'w_qdq': partial(self.w_qdq, wquantizer=self.wquantizer)}
        if mode in _REALQUANT_MODES:
            return {'w_q': partial(self.w_q, wquantizer=self.wquantizer), 'quant_config': self.quant_config}
        raise NotImplementedError(f'mode {mode}')

    # -- qparams registered on the layers ---------------------------------------------------------------------
    @torch.no_grad()
    def collect_block_qparams(self, named_linears):
        """base_blockwise_quantization.py:348-376 over a {name: Linear} dict (there: model.get_block_linears(block))."""
        for m in named_linears.values():
            args = {k: getattr(m, f'buf_{k}') for k in ('lowbound_factor', 'upbound_factor') if hasattr(m, f'buf_{k}')}
            if m.weight.data.dtype == torch.float8_e4m3fn:
                weight = weight_cast_to_bf16(m.weight.data, m.weight_scale_inv.data, self.fp8_block_size).to(torch.bfloat16)
            else:
                weight = m.weight.data
            _, scales, zeros, max_int, min_int = self.wquantizer.get_tensor_qparams(weight, args=args)
            m.register_buffer('buf_scales', scales.detach())
            m.register_buffer('buf_zeros', zeros.detach())
            m.register_buffer('buf_qmax', torch.as_tensor(max_int).clone().to(weight.device))
            m.register_buffer('buf_qmin', torch.as_tensor(min_int).clone().to(weight.device))

    @torch.no_grad()
    def register_act_qparams(self, layers_dict, act_tensors):
        """base_blockwise_quantization.py:590-611 on one GPU (no all-reduce of the scales)."""
        scales_list, zeros_list, qmin_list, qmax_list = self.aquantizer.get_batch_tensors_qparams(act_tensors)
        for i, (scales, zeros, qmin, qmax) in enumerate(zip(scales_list, zeros_list, qmin_list, qmax_list)):
            for layer in layers_dict.values():
                if not is_linear_like(layer):
                    continue
                layer.register_buffer(f'buf_act_scales_{i}', scales.cuda())
                layer.register_buffer(f'buf_act_zeros_{i}', zeros.cuda())
                layer.register_buffer(f'buf_act_qmin_{i}', qmin.cuda())
                layer.register_buffer(f'buf_act_qmax_{i}', qmax.cuda())

    # -- rtn.py:14-29 -----------------------------------------------------------------------------------------
    @torch.no_grad()
    def subset_transform(self, subset, input_feat, subset_kwargs):
        pass
