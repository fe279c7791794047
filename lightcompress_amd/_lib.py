"""ctypes binding of liblcq.so — the only way the Python layer reaches the GPU.

There is deliberately no CPU fallback: if the shared object is missing or a
tensor is not on the GPU, calls raise.
"""
from __future__ import annotations

import ctypes as C
import re
from pathlib import Path

import torch

_PKG = Path(__file__).resolve().parent
LIB_PATH = _PKG / 'liblcq.so'
HEADER = _PKG.parent / 'include' / 'lcq.h'

# constants mirrored from include/lcq.h
F32, BF16, F16 = 0, 1, 2
CODE_NONE, CODE_U8, CODE_I8, CODE_I32, CODE_SAME, CODE_F32, CODE_FP8, CODE_CT4 = range(8)
FLAG_SYM, FLAG_NO_ROUND_ZP, FLAG_STATIC, FLAG_SCALAR_QP = 1, 2, 4, 8
FLAG_TIE_EVEN, FLAG_NO_SUBNORMALS, FLAG_DQ_F32 = 16, 32, 64
FLAG_RANGE_BF16, FLAG_SCALE_F32, FLAG_ROW_QP = 128, 256, 512
FLAG_ROWS16 = 4096
FLAG_RANGE_F16 = 8192

_ERR = {-1: 'invalid argument', -2: 'misaligned pointer', -3: 'unsupported dtype', -4: 'kernel launch failed',
        -5: 'workspace too small', -6: 'input larger than the entry point\'s stated maximum'}


class LcqError(RuntimeError):
    pass


_lib = None


def declared_symbols() -> list[str]:
    """Names of every function the headers under include/ declare (lcq.h: the boundary; lcq_bench.h: benchmark aids)."""
    names = set()
    for header in sorted(HEADER.parent.glob('*.h')):
        text = re.sub(r'/\*.*?\*/', '', header.read_text(), flags=re.S)
        names.update(re.findall(r'\b(lcq_[a-z0-9_]+)\s*\(', text))
    return sorted(names)


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise LcqError(f'{LIB_PATH} is missing: run `python -m lightcompress_amd.build` '
                           '(there is no CPU fallback for this path)')
        _lib = C.CDLL(str(LIB_PATH))
        for name in declared_symbols():
            fn = getattr(_lib, name)
            fn.restype = C.c_int64 if name.endswith('_workspace_bytes') else C.c_int
    return _lib


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    if dt == torch.float16:
        return F16
    raise LcqError(f'unsupported dtype {dt}')


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    if t is None:
        return C.c_void_p(0)
    if not t.is_cuda:
        raise LcqError('liblcq operates on GPU tensors only (no CPU fallback)')
    if not t.is_contiguous():
        raise LcqError('tensor must be contiguous')
    return C.c_void_p(t.data_ptr())


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def check(rc: int, what: str):
    if rc != 0:
        raise LcqError(f'{what} failed: {_ERR.get(rc, rc)} ({rc})')


def i64(v):
    return C.c_int64(int(v))


def f32(v):
    return C.c_float(float(v))


def i32(v):
    return C.c_int(int(v))
