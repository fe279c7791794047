"""CPU-side checks of the C-ABI library: it loads, exports every symbol the
header declares, and the Python layer refuses to run without a GPU."""
import ctypes

import pytest
import torch

from lightcompress_amd import _lib


def test_library_exports_every_declared_symbol():
    names = _lib.declared_symbols()
    assert len(names) >= 10
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for n in names:
        assert hasattr(lib, n), n


def test_cpu_tensors_are_refused_not_emulated():
    from lightcompress_amd import FloatQuantizer, IntegerQuantizer
    from lightcompress_amd.module_utils import VllmRealQuantLinear
    q = IntegerQuantizer(4, False, 'per_group', group_size=128)
    with pytest.raises(_lib.LcqError):
        q.fake_quant_weight_dynamic(torch.randn(4, 128))
    with pytest.raises(_lib.LcqError):
        q.real_quant_weight_dynamic(torch.randn(4, 128))
    f = FloatQuantizer('e4m3', True, 'per_channel', use_qtorch=True)
    with pytest.raises(_lib.LcqError):
        f.fake_quant_weight_dynamic(torch.randn(4, 128))
    with pytest.raises(_lib.LcqError):
        VllmRealQuantLinear.pack(torch.zeros(2, 8, dtype=torch.int32), torch.ones(2, 1), {'weight': {'bit': 4}})


def test_constructor_surface_matches_reference():
    from lightcompress_amd import FloatQuantizer, IntegerQuantizer
    q = IntegerQuantizer(4, False, 'per_group', group_size=128)
    assert q.qmin.dtype == torch.float32 and float(q.qmin) == 0.0 and int(q.qmax) == 15 and q.qmax.dtype == torch.int64
    q = IntegerQuantizer(8, True, 'per_channel')
    assert int(q.qmin) == -128 and int(q.qmax) == 127 and q.qmin.dtype == torch.int64
    q = IntegerQuantizer(4, True, 'per_tensor', int_range=[-7, 7])
    assert int(q.qmin) == -7
    f = FloatQuantizer('e4m3', False, 'per_channel', use_qtorch=True)
    assert f.sym is True and float(f.qmax) == 448.0 and f.e_bits == 4 and f.m_bits == 3
    assert float(FloatQuantizer('e5m2', True, 'per_tensor', use_qtorch=True).qmax) == 57344.0
    assert float(FloatQuantizer('e2m1', True, 'per_tensor', use_qtorch=True).qmax) == 6.0
    with pytest.raises(ValueError):
        IntegerQuantizer(4, False, 'per_group', group_size=128).reshape_tensor(torch.zeros(2, 130))


def test_mirror_classes_keep_the_reference_method_names():
    """The method names of the reference classes on the path (quant.py, gptq.py, awq.py, auto_clip.py, rtn.py,
    base_blockwise_quantization.py, module_utils.py), as listed from its sources: every one is there on the mirror."""
    import lightcompress_amd.quant as quant
    from lightcompress_amd.auto_clip import AutoClipper
    from lightcompress_amd.awq import Awq
    from lightcompress_amd.blockwise import ScaleFolding
    from lightcompress_amd.gptq import GPTQ
    from lightcompress_amd.module_utils import (AutoawqRealQuantLinear, EffcientFakeQuantLinear, FakeQuantLinear,
                                                SglRealQuantLinear, VllmRealQuantLinear)
    from lightcompress_amd.rtn import RTN
    names = {
        quant.IntegerQuantizer: 'get_tensor_range get_minmax_range get_mse_range get_learnable_range get_minmax_stats '
                                'get_static_minmax_range get_norm get_quantization_error get_static_moving_minmax_range '
                                'get_qparams get_batch_tensors_qparams optimize_weights_proximal reshape_tensor restore_tensor '
                                'get_hqq_qparams get_tensor_qparams quant dequant quant_dequant fake_quant_act_static '
                                'fake_quant_act_dynamic fake_quant_weight_static fake_quant_weight_dynamic '
                                'real_quant_weight_static real_quant_weight_dynamic',
        quant.FloatQuantizer: 'get_float_qparams get_tensor_qparams quant dequant quant_dequant fake_quant_act_static '
                              'fake_quant_act_dynamic fake_quant_weight_static fake_quant_weight_dynamic '
                              'real_quant_weight_static real_quant_weight_dynamic',
        GPTQ: 'add_quant_config hessian_sorting subset_transform layer_transform initialize_qparams_and_prepare_weights '
              'process_hessian_and_weights update_layer_with_transformed_weights weight_transform add_batch layer_init '
              'subset_init split_qparams merge_qparams search_column_qparams search_layer_qparams search_group_qparams '
              'update_model_qparams w_q w_qdq free ready',
        Awq: 'scaling_weight get_weight_scale get_act_scale get_scales inspect_module_forward get_original_out '
             'calculate_loss fake_quantize_weight fake_quantize_input search_scale_subset subset_transform apply_scale '
             'scale_fc_fc scale_ln_fcs scaling_input update_input_feat repeat_gqa_scales',
        AutoClipper: 'run auto_clip_layer apply_clip get_clip_factor fake_quantize_weight fake_quantize_input',
        ScaleFolding: 'apply_scale scale_fc_fc scale_ln_fcs scaling_input update_input_feat repeat_gqa_scales',
        RTN: 'set_quant_config w_qdq w_q a_qdq get_replacement_params collect_block_qparams register_act_qparams '
             'subset_transform',
        VllmRealQuantLinear: 'new quant_pack pack forward', SglRealQuantLinear: 'new quant_pack pack forward',
        AutoawqRealQuantLinear: 'new quant_pack gemm_pack forward',
        FakeQuantLinear: 'new get_func_name forward', EffcientFakeQuantLinear: 'new get_func_name forward',
    }
    missing = [f'{cls.__name__}.{n}' for cls, ns in names.items() for n in ns.split() if not hasattr(cls, n)]
    assert not missing, missing


def test_rtn_picks_the_quantizers_like_set_quant_config():
    from lightcompress_amd import FloatQuantizer, IntegerQuantizer, Weight48IntegerQuantizer
    from lightcompress_amd.rtn import RTN, select_quantizer
    assert select_quantizer({'bit': 4}) is IntegerQuantizer and select_quantizer({'bit': 48}) is Weight48IntegerQuantizer
    assert select_quantizer({'bit': 'e4m3', 'quant_type': 'float-quant'}) is FloatQuantizer
    with pytest.raises(ValueError):
        select_quantizer({'bit': 4, 'quant_type': 'other'})
    cfg = {'weight': dict(bit=8, symmetric=True, granularity='per_channel'),
           'act': dict(bit=8, symmetric=True, granularity='per_tensor', static=True),
           'special': dict(weight_clip=True, clip_version='v1')}
    rtn = RTN(cfg)
    assert rtn.act_static and cfg['act']['calib_algo'] == 'static_minmax' and not rtn.w_only
    assert rtn.auto_clipper.clip_version == 'v1' and rtn.aquantizer.calib_algo == 'static_minmax'
