"""Export config writers and deploy containers (host logic, no GPU): the JSON the loaders of vLLM / SGLang
(compressed-tensors, fp8) and AutoAWQ read, and the buffer names of the real-quant Linear containers."""
import json
import types

import torch

from lightcompress_amd import export as E


class Cfg(dict):
    """attribute + item access like the reference's EasyDict"""
    def __getattr__(self, k):
        try:
            return self[k]
        except KeyError as e:
            raise AttributeError(k) from e


def cfg(**kw):
    return Cfg({k: cfg(**v) if isinstance(v, dict) else v for k, v in kw.items()})


def _write(tmp_path, content):
    (tmp_path / 'config.json').write_text(json.dumps(content))
    return str(tmp_path)


def _read(tmp_path):
    return json.loads((tmp_path / 'config.json').read_text())


MODEL = types.SimpleNamespace(skip_layer_name=lambda: ['lm_head'])


def test_autoawq_config(tmp_path):
    c = cfg(quant=dict(weight=dict(bit=4, symmetric=False, granularity='per_group', group_size=128, pack_version='gemm_pack')))
    path = _write(tmp_path, {'model_type': 'llama', 'quantization_config': {'old': 1}})
    E.update_autoawq_quant_config(c, path)
    out = _read(tmp_path)
    assert out['model_type'] == 'llama'
    assert out['quantization_config'] == {'bits': 4, 'group_size': 128, 'modules_to_not_convert': None, 'quant_method': 'awq',
                                          'version': 'gemm', 'zero_point': True}
    c.quant.weight['granularity'] = 'per_channel'
    E.update_autoawq_quant_config(c, path)
    assert _read(tmp_path)['quantization_config']['group_size'] == -1


def test_vllm_compressed_tensors_int4_packed(tmp_path):
    c = cfg(quant=dict(weight=dict(bit=4, symmetric=True, granularity='per_group', group_size=128, need_pack=True)))
    path = _write(tmp_path, {'quantization_config': {'stale': True}, 'hidden_size': 8})
    E.update_vllm_quant_config(MODEL, c, path)
    out = _read(tmp_path)
    assert 'quantization_config' not in out and out['hidden_size'] == 8
    cc = out['compression_config']
    assert cc['format'] == 'pack-quantized' and cc['quant_method'] == 'compressed-tensors' and cc['ignore'] == ['lm_head']
    g = cc['config_groups']['group_0']
    assert g['targets'] == ['Linear'] and g['input_activations'] is None
    assert g['weights'] == {'dynamic': False, 'group_size': 128, 'num_bits': 4, 'observer': 'minmax', 'observer_kwargs': {},
                            'strategy': 'group', 'symmetric': True, 'type': 'int'}


def test_vllm_w8a8_int_and_fp8_variants(tmp_path):
    c = cfg(quant=dict(weight=dict(bit=8, symmetric=True, granularity='per_channel'),
                       act=dict(bit=8, symmetric=True, granularity='per_token')))
    path = _write(tmp_path, {})
    E.update_vllm_quant_config(MODEL, c, path)
    g = _read(tmp_path)['compression_config']
    assert g['format'] == 'int-quantized'
    a = g['config_groups']['group_0']['input_activations']
    assert a['dynamic'] is True and a['num_bits'] == 8 and a['strategy'] == 'token' and a['type'] == 'int'
    assert g['config_groups']['group_0']['weights']['strategy'] == 'channel'
    # static fp8
    c = cfg(quant=dict(weight=dict(bit='e4m3', symmetric=True, granularity='per_tensor', quant_type='float-quant'),
                       act=dict(bit='e4m3', symmetric=True, granularity='per_tensor', quant_type='float-quant', static=True)))
    path = _write(tmp_path, {'x': 1})
    E.update_vllm_quant_config(MODEL, c, path)
    assert _read(tmp_path)['quantization_config'] == {'activation_scheme': 'static', 'ignored_layers': [['lm_head']],
                                                     'quant_method': 'fp8'}
    # dynamic fp8 with block-wise weights
    c = cfg(quant=dict(weight=dict(bit='e4m3', symmetric=True, granularity='per_block', block_size=128, quant_type='float-quant'),
                       act=dict(bit='e4m3', symmetric=True, granularity='per_group', group_size=128, quant_type='float-quant')))
    E.update_vllm_quant_config(MODEL, c, path)
    assert _read(tmp_path)['quantization_config'] == {'activation_scheme': 'dynamic', 'fmt': 'e4m3', 'quant_method': 'fp8',
                                                     'weight_block_size': [128, 128]}
    # weight-only fp8
    c = cfg(quant=dict(weight=dict(bit='e4m3', symmetric=True, granularity='per_channel', quant_type='float-quant')))
    E.update_vllm_quant_config(MODEL, c, path)
    assert _read(tmp_path)['compression_config']['format'] == 'float-quantized'
    assert _read(tmp_path)['compression_config']['config_groups']['group_0']['weights']['num_bits'] == 8


def test_container_buffer_names():
    from lightcompress_amd.module_utils import AutoawqRealQuantLinear, VllmRealQuantLinear
    w = torch.zeros(4, 2, dtype=torch.int32)
    s = torch.ones(4, 1, dtype=torch.float16)
    m = VllmRealQuantLinear(w, None, s, None, True, 'weight_scale')
    assert set(dict(m.named_buffers())) == {'weight_packed', 'weight_scale'} and m.bias is None and m.input_scale is None
    m = VllmRealQuantLinear(w, torch.zeros(4), s, torch.ones(1), False, 'weight_scale_inv')
    assert set(dict(m.named_buffers())) == {'weight', 'weight_scale_inv', 'bias', 'input_scale'}
    a = AutoawqRealQuantLinear(w, None, s, w.clone())
    assert set(dict(a.named_buffers())) == {'qweight', 'scales', 'qzeros'}
    assert set(AutoawqRealQuantLinear(w, None, s, None).state_dict()) == {'qweight', 'scales'}
