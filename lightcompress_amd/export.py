"""`quantization_config` / `compression_config` entries of an exported checkpoint's config.json.

Same output as ``update_autoawq_quant_config`` (llmc/utils/export_autoawq.py:4-30) and
``update_vllm_quant_config`` (llmc/utils/export_vllm.py:4-125) of ModelTC/LightCompress, so that the packed
tensors written by ``lightcompress_amd.module_utils`` load in AutoAWQ and in vLLM / SGLang (compressed-tensors or
the native fp8 method).  ``config`` is the reference's run configuration (attribute and item access, e.g. an
EasyDict); ``model.skip_layer_name()`` lists the layers left unquantized.
"""
from __future__ import annotations

import json
import os


def _rewrite(save_quant_path, edit):
    path = os.path.join(save_quant_path, 'config.json')
    with open(path, 'r') as f:
        cfg = json.load(f)
    edit(cfg)
    with open(path, 'w') as f:
        json.dump(cfg, f, indent=4)


def _get(node, key, default=None):
    return node.get(key, default) if hasattr(node, 'get') else getattr(node, key, default)


def update_autoawq_quant_config(config, save_quant_path):
    w = config.quant.weight
    entry = {
        'bits': w.bit,
        'group_size': w.group_size if w.granularity == 'per_group' else -1,
        'modules_to_not_convert': None,
        'quant_method': 'awq',
        'version': w.pack_version.split('_')[0],
        'zero_point': not w.symmetric,
    }

    def edit(cfg):
        cfg.pop('quantization_config', None)
        cfg['quantization_config'] = entry
    _rewrite(save_quant_path, edit)


def update_vllm_quant_config(model, config, save_quant_path, vllm_quant_method='compressed-tensors'):
    quant = config.quant
    w = quant.weight
    has_act = 'act' in quant
    w_type = _get(w, 'quant_type', 'int-quant')
    a_type = None
    if has_act:
        a_type = _get(quant.act, 'quant_type', 'int-quant')
        assert a_type == w_type
    a_bits = None

    if a_type == 'float-quant':
        # native fp8 checkpoints: static per-tensor activations, or dynamic with block-wise weights
        if _get(quant.act, 'static', False):
            entry = {'activation_scheme': 'static', 'ignored_layers': [model.skip_layer_name()], 'quant_method': 'fp8'}
            _rewrite(save_quant_path, lambda cfg: cfg.__setitem__('quantization_config', entry))
            return
        if _get(w, 'granularity', 'per_block'):
            entry = {'activation_scheme': 'dynamic', 'fmt': 'e4m3', 'quant_method': 'fp8',
                     'weight_block_size': [w.block_size, w.block_size]}
            _rewrite(save_quant_path, lambda cfg: cfg.__setitem__('quantization_config', entry))
            return
        fmt, kind, w_bits, a_bits = 'float-quantized', 'float', 8, 8
    elif _get(w, 'need_pack', False):
        fmt, kind, w_bits = 'pack-quantized', 'int', w.bit
    elif w_type == 'float-quant':
        fmt, kind, w_bits = 'float-quantized', 'float', 8
    else:
        fmt, kind, w_bits = 'int-quantized', 'int', w.bit
        if has_act:
            a_bits = quant.act.bit

    per_group = w.granularity == 'per_group'
    dynamic = (not quant.act.static) if has_act and 'static' in quant.act else True
    acts = None
    if has_act:
        acts = {'dynamic': dynamic, 'group_size': None, 'num_bits': a_bits, 'observer': 'minmax', 'observer_kwargs': {},
                'strategy': 'token' if quant.act.granularity == 'per_token' else 'tensor',
                'symmetric': quant.act.symmetric, 'type': kind}
    weights = {'dynamic': False, 'group_size': w.group_size if per_group else None, 'num_bits': w_bits,
               'observer': 'minmax', 'observer_kwargs': {}, 'strategy': 'group' if per_group else 'channel',
               'symmetric': w.symmetric, 'type': kind}
    entry = {'config_groups': {'group_0': {'targets': ['Linear'], 'input_activations': acts, 'weights': weights}},
             'format': fmt, 'ignore': model.skip_layer_name(), 'quant_method': vllm_quant_method}

    def edit(cfg):
        if w_type == 'int-quant':
            cfg.pop('quantization_config', None)
        cfg['compression_config'] = entry
    _rewrite(save_quant_path, edit)
