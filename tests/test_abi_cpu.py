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
